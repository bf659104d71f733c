"""Natatar without a GPU: its configuration, plan, checkpoint names and caches, and the plain implementation held
against itself (what the streams, the rotation of neighbours, the matrix memory, the decays per channel and the
router with groups do)."""

import copy
import math

import pytest
import torch

from tests import plain_natatar as plain
from tests.natatar_cases import CASES, random_weights

F = torch.float64


def parts_of(raw):
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.models.decoder import DecoderModel

    arch = architecture_for(raw)
    config = arch.parse_config(raw)
    return arch, config, DecoderModel(arch.build_plan(config), torch.float32, "cpu")


@pytest.mark.parametrize("case", sorted(CASES))
def test_configuration_plan_and_names(case):
    raw = CASES[case]
    arch, config, model = parts_of(raw)
    assert arch.name == "Natatar" and arch.parse_config(config.to_dict()) == config
    plan = model.plan
    assert [r.layer for r in plan.run] == list(range(len(raw["layers"]))) and all(r.cache is None and r.writes for r in plan.run)
    assert plan.tied_head and plan.embedding_scale == (raw.get("embedding") or {}).get("scale", 1.0)
    assert plan.final_norm.offset == 1.0
    for i, block in enumerate(plan.layers):
        assert block.arrangement == "streams_prenorm" and block.streams == raw.get("streams", 0)
        assert block.residual_scale == raw.get("residual_mult", 1.0)
        assert (block.streams_first, block.streams_last) == (i == 0, i == len(plan.layers) - 1)
    weights = random_weights(raw, seed=1)
    shapes = arch.checkpoint_shapes(config)
    assert set(shapes) == set(weights) and all(tuple(weights[k].shape) == tuple(v[0]) for k, v in shapes.items())
    from atomserve_amd.weights.loader import as_stack

    used = [t.name for target in model.weight_decls() for t in as_stack(arch.checkpoint_map(config)[target]).parts]
    assert len(used) == len(set(used)), "no tensor of the checkpoint is read twice"
    assert set(weights) - set(used) <= arch.ignored(config) and set(used) <= set(weights) and not set(used) & arch.ignored(config)
    assert model.capturable


def test_which_layer_keeps_values_and_which_mix_them():
    raw = CASES["two_streams"]
    arch, config, model = parts_of(raw)
    kinds = [block.mixer.cores[0].value_mix if block.mixer.kind == "joined" else None for block in model.plan.layers]
    assert kinds == [None, "first", "none", "none", "later"]
    assert arch.ignored(config) == {"l1.mix.vmix", "l2.mix.vmix"}, "the first mixing layer's own weight is stored and unused"
    assert "layers.4.mixer.c0.value_mix" in model.weight_decls() and "layers.1.mixer.c0.value_mix" not in model.weight_decls()


def test_caches_pages_for_attentions_and_slots_for_states():
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.parts.base import PagedCacheRequest, StateCacheRequest

    raw = CASES["two_streams"]
    _, _, model = parts_of(raw)
    requests = model.cache_requests()
    paged = {k: v for k, v in requests.items() if isinstance(v, PagedCacheRequest)}
    states = {k: v for k, v in requests.items() if isinstance(v, StateCacheRequest)}
    assert sorted(paged) == [(1, "0.pages"), (2, "0.pages"), (3, "0.pages"), (4, "0.pages")]
    assert (paged[(1, "0.pages")].num_kv_heads, paged[(1, "0.pages")].head_dim) == (2, 32)  # 16 and 24 in steps of 32
    assert (paged[(2, "0.pages")].num_kv_heads, paged[(2, "0.pages")].head_dim) == (3, 8)
    assert all(p.window == 0 for p in paged.values())
    assert states[(0, "state")].shape == (4, 24, 16) and states[(0, "conv")].shape == (2, 2 * 2 * 24 + 4 * 16)
    assert states[(3, "1.state")].shape == (3, 8, 24) and states[(3, "1.normaliser")].shape == (3, 8)
    assert states[(3, "1.maximum")].shape == (3,) and all(s.dtype == torch.float32 for s in states.values())
    manager = CacheManager(requests, 16, 40, 2)
    assert not manager.prefix_reuse_possible  # what a state holds cannot be taken over from another request's pages
    a, b = manager.new_request(), manager.new_request()
    assert manager.reserve(a, 0, 40) and manager.reserve(b, 0, 100)
    assert a.state_slot != b.state_slot
    manager.release(a)
    c = manager.new_request()
    assert c.state_slot == a.state_slot and manager.reserve(c, 0, 33)
    manager.release(b)
    manager.release(c)
    assert manager.num_free == manager.num_blocks


def test_what_the_configuration_refuses_and_completes():
    from atomserve_amd.config.model_config import ConfigError, NatatarConfig

    raw = CASES["two_streams"]
    for change, needle in (
        (lambda r: r["layers"][0].update(type="delta"), "type"),
        (lambda r: r["layers"][0]["mlp"].update(kind="dense"), "kind"),
        (lambda r: r["layers"][1]["mixer"].pop("scale"), "scale"),
        (lambda r: r["layers"][3]["mixer"]["left"]["rot"].update(dims=34), "rot"),
        (lambda r: r["layers"][3]["mixer"]["right"].update(gate_cap=0.0), "gate_cap"),
        (lambda r: r["layers"][4]["mixer"].update(vdim=8), "mix values"),
        (lambda r: r["layers"][4]["mixer"].update(vdim=12, kv_heads=3, heads=3), "mix values"),
        (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
        (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=6), "groups"),
        (lambda r: r["layers"][1]["mixer"].update(heads=3), "kv_heads"),
        (lambda r: r["norm"].pop("eps"), "eps"),
    ):
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError, match=needle):
            NatatarConfig.from_dict(broken)
    # ranks that config.json does not name come from the tensors' shapes; without either there is no plan
    bare = copy.deepcopy(raw)
    bare["layers"][0]["mixer"].pop("decay_rank")
    bare["layers"][0]["mixer"].pop("gate_rank")
    arch, _, _ = parts_of(raw)
    config = arch.parse_config(bare)
    with pytest.raises(ConfigError, match="ranks"):
        arch.build_plan(config)
    shapes = {"l0.mix.a1": (5, 96), "l0.mix.g1": (7, 96)}
    assert arch.complete(config, shapes.get) == arch.parse_config(raw)


def test_shapes_are_read_from_a_file_header(tmp_path):
    from safetensors.torch import save_file

    from atomserve_amd.weights.loader import checkpoint_shapes_of

    save_file({"a.b": torch.zeros(3, 5), "s": torch.zeros(())}, str(tmp_path / "model.safetensors"))
    shape_of = checkpoint_shapes_of(str(tmp_path))
    assert shape_of("a.b") == (3, 5) and shape_of("s") == () and shape_of("absent") is None


# ---- the plain implementation against itself ----------------------------------------------------------------------


def test_one_stream_with_unit_coefficients_is_the_plain_residual_sum():
    raw = copy.deepcopy(CASES["plain_sums"])
    weights = random_weights(raw, seed=5)
    ids = list(range(3, 23))
    want = plain.logits(raw, weights, ids)
    raw["streams"] = 1
    for i, layer in enumerate(raw["layers"]):
        for q in (1, 2) if layer["mlp"] is not None else (1,):
            weights[f"l{i}.hc{q}.in"], weights[f"l{i}.hc{q}.out"], weights[f"l{i}.hc{q}.mix"] = torch.ones(1), torch.ones(1), torch.ones(1, 1)
    assert torch.allclose(plain.logits(raw, weights, ids), want, atol=1e-6)


def test_streams_write_from_the_old_streams_all_at_once():
    xs = torch.randn(3, 4, 5, dtype=F)
    M, c, y = torch.randn(3, 3, dtype=F), torch.randn(3, dtype=F), torch.randn(4, 5, dtype=F)
    new = plain.streams_write(xs, M, c, 0.45, y)
    for r in range(3):
        want = sum(M[s, r] * xs[s] for s in range(3)) + 0.45 * c[r] * y
        assert torch.allclose(new[r], want)
    assert torch.allclose(plain.streams_read(xs, c), sum(c[s] * xs[s] for s in range(3)))


def test_a_later_token_changes_nothing_before_it():
    raw = CASES["two_streams"]
    weights = random_weights(raw, seed=2)
    ids = list(range(10, 40))
    other = ids[:20] + [7] + ids[21:]
    a, b = plain.logits(raw, weights, ids), plain.logits(raw, weights, other)
    assert torch.equal(a[:20], b[:20]) and not torch.allclose(a[20:], b[20:])


def test_neighbours_turn_by_their_positions_difference():
    rot = {"dims": 6, "base": 100.0}
    q, k = torch.randn(1, 1, 10, dtype=F), torch.randn(1, 1, 10, dtype=F)

    def score(i, j):
        return float((plain.rotate_neighbours(q, torch.tensor([i]), rot) * plain.rotate_neighbours(k, torch.tensor([j]), rot)).sum())

    assert abs(score(17, 5) - score(112, 100)) < 1e-9 and abs(score(17, 5) - score(17, 6)) > 1e-6
    turned = plain.rotate_neighbours(q, torch.tensor([9]), rot)
    assert torch.equal(turned[..., 6:], q[..., 6:]), "coordinates beyond rot.dims pass unchanged"
    f0 = 9 * 100.0 ** (-2 * 1 / 6)  # pair 1 = coordinates (2, 3)
    assert abs(float(turned[0, 0, 2]) - float(q[0, 0, 2] * math.cos(f0) - q[0, 0, 3] * math.sin(f0))) < 1e-12
    assert abs(float(turned[0, 0, 3]) - float(q[0, 0, 3] * math.cos(f0) + q[0, 0, 2] * math.sin(f0))) < 1e-12


def test_stretched_frequencies_keep_the_fast_and_divide_the_slow():
    rot = {"dims": 32, "base": 10000.0, "scaling": {"factor": 8.0, "original": 512, "fast": 16.0, "slow": 1.0}}
    f, mag = plain.stretched_frequencies(rot)
    plain_f = 10000.0 ** (-2.0 * torch.arange(16, dtype=F) / 32)
    assert torch.allclose(f[:3], plain_f[:3]) and torch.allclose(f[-3:], plain_f[-3:] / 8.0)
    assert abs(mag - (0.1 * math.log(8.0) + 1.0)) < 1e-12
    assert plain.stretched_frequencies({"dims": 32, "base": 10000.0})[1] == 1.0


def test_matrix_memory_first_token_and_forgetting():
    """The first token of a sequence: m = max(f + 0, i); with i = 0 and f < 0 this is 0, S = k v^T, n = k, so the output
    is (k . q) v / (max(|k . q|, 1) + 1e-6).  A forget gate of minus infinity makes every token a first token."""
    H, D, E = 2, 4, 3
    q, k, v = torch.randn(5, H, D, dtype=F), torch.randn(5, H, D, dtype=F), torch.randn(5, H, E, dtype=F)
    zero, never = torch.zeros(5, H, dtype=F), torch.full((5, H), -50.0, dtype=F)
    out = plain.matrix_memory_scan(q, k, v, zero, never)
    kq = (k * q).sum(-1, keepdim=True)
    assert torch.allclose(out, kq * v / (torch.maximum(kq.abs(), torch.ones_like(kq)) + 1e-6), atol=1e-9)
    # a large input gate: the maximum follows it, and e^(-m) no longer bounds the denominator
    big = torch.full((5, H), 20.0, dtype=F)
    out = plain.matrix_memory_scan(q[:1], k[:1], v[:1], big[:1], never[:1])
    assert torch.allclose(out, kq[:1] * v[:1] / (kq[:1].abs().clamp_min(math.exp(-20.0)) + 1e-6), atol=1e-9)


def test_delta_rule_reads_back_what_it_wrote_and_decays_by_channel():
    H, D, E = 1, 4, 3
    k = torch.zeros(3, H, D, dtype=F)
    k[0, 0, 1] = k[1, 0, 2] = 1.0
    k[2, 0, 1] = 1.0
    v = torch.randn(3, H, E, dtype=F)
    q = k.clone()
    one = torch.ones(3, H, dtype=F)
    g = torch.ones(3, H, D, dtype=F)
    out = plain.channel_delta_scan(q, k, v, one, g)
    assert torch.allclose(out[0], v[0]) and torch.allclose(out[1], v[1]) and torch.allclose(out[2], v[2]), "beta 1 replaces what a key holds"
    g[1:, 0, 1] = 0.5  # channel 1 decays at tokens 1 and 2, channel 2 does not
    half = torch.full((3, H), 0.0, dtype=F)
    half[0] = 1.0  # only the first token writes
    out = plain.channel_delta_scan(q, k, v, half, g)
    assert torch.allclose(out[2], 0.25 * v[0]) and torch.allclose(out[1], torch.zeros_like(v[1]))


def test_router_keeps_the_best_groups_and_breaks_ties_downwards():
    scores = torch.tensor([[0.05, 0.30, 0.10, 0.20, 0.25, 0.10]], dtype=F)
    assert plain.grouped_choice(scores, 2, 1, 1).tolist() == [[1, 4]]
    assert plain.grouped_choice(scores, 2, 3, 1).tolist() == [[1, 0]], "only the group of the largest score"
    assert plain.grouped_choice(scores, 3, 3, 2).tolist() == [[1, 4, 5]], "groups (0, 1) and (4, 5); 0.10 of expert 2 is shut out"
    tie = torch.tensor([[0.25, 0.25, 0.25, 0.25]], dtype=F)
    assert plain.grouped_choice(tie, 2, 2, 1).tolist() == [[0, 1]]


def test_experts_weigh_scores_times_the_factor_without_renormalising():
    raw = {"router": {"experts": 3, "top": 3, "scale": 2.5}, "expert": {"ff": 4}}
    g = torch.Generator().manual_seed(0)
    W = {"x.router": torch.randn(3, 6, generator=g, dtype=F)}
    for e in range(3):
        W[f"x.e{e}.gate"], W[f"x.e{e}.up"], W[f"x.e{e}.down"] = (torch.randn(4, 6, generator=g, dtype=F), torch.randn(4, 6, generator=g, dtype=F),
                                                                   torch.randn(6, 4, generator=g, dtype=F))  # fmt: skip
    h = torch.randn(2, 6, generator=g, dtype=F)
    out = plain.experts(h, W, "x.", raw, False)
    s = torch.softmax(h @ W["x.router"].t(), -1)
    want = sum(2.5 * s[:, e : e + 1] * ((torch.nn.functional.silu(h @ W[f"x.e{e}.gate"].t()) * (h @ W[f"x.e{e}.up"].t())) @ W[f"x.e{e}.down"].t())
               for e in range(3))  # fmt: skip
    assert torch.allclose(out, want)


def test_norms_add_one_to_the_layers_gains_and_not_to_the_heads():
    x = torch.randn(3, 8, dtype=F)
    w = torch.randn(8, dtype=F) * 0.1
    unit = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose(plain.offset_norm(x, w, 1e-5), unit * (1 + w)) and torch.allclose(plain.plain_norm(x, w, 1e-5), unit * w)
