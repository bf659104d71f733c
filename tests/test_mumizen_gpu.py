"""Mumizen on the GPU against the plain implementation (tests/plain_mumizen.py): each mechanism alone, and whole
models of several shapes stepped whole, token by token, in portions down to two tokens, in mixed batches with pages
and state slots used again, and through the engine's scheduler.  Configurations and weights are made here; where
random weights would hide a fault (a far key among hundreds, a page's border, a slot that another request left
full) the inputs are made so that it shows."""

import copy
import json
import math
import os

import pytest
import torch

from tests import plain_mumizen as plain
from tests import replay_cases as rc
from tests.mumizen_cases import CASES, random_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
I32 = torch.int32


def build_model(raw, weights, dtype):
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.models.decoder import DecoderModel
    from atomserve_amd.weights.loader import DictSource, bind_checkpoint

    arch = architecture_for(raw)
    config = arch.parse_config(raw)
    model = DecoderModel(arch.build_plan(config), DTYPES[dtype], DEV)
    bind_checkpoint(model, arch, config, DictSource(weights))
    return model


def make_replay(raw, weights, dtype, max_tokens, block_size=16, max_live=4):
    from atomserve_amd.engine.replay import Replay

    return Replay("", dtype, max_tokens, device=DEV, block_size=block_size, max_live=max_live, model=build_model(raw, weights, dtype))


class Against:
    """Engine - plain, row by row, beside what rounding to bfloat16 alone does to the plain model at the same rows."""

    def __init__(self):
        self.err, self.noise, self.scale = [], [], 1.0

    def add(self, got, exact, rounded=None):
        got, exact = got.reshape(-1, exact.shape[-1]), exact.reshape(-1, exact.shape[-1])
        self.err += (got - exact).pow(2).mean(-1).sqrt().tolist()
        if rounded is not None:
            self.noise += (rounded.reshape(exact.shape) - exact).pow(2).mean(-1).sqrt().tolist()
        self.scale = max(self.scale, float(exact.abs().max()))

    def take(self, other):
        self.err += other.err
        self.noise += other.noise
        self.scale = max(self.scale, other.scale)

    def check(self, dtype, what=""):
        """32-bit: rounding of float32 only, at every row.  bfloat16: the rows' errors as a distribution against what
        rounding the stored activations moves the plain model itself at the same rows (a token whose router logits lie
        within rounding of each other may take another expert in either model; such rows stand out in both)."""
        assert self.err
        err = torch.tensor(self.err)
        if dtype == "float32":
            assert float(err.max()) <= 3e-5 * self.scale, f"{what}: {float(err.max()):.3e} against |logits| {self.scale:.3e}"
            return
        noise = torch.tensor(self.noise)
        mid, high = (float(err.median()), float(noise.median())), (float(err.quantile(0.9)), float(noise.quantile(0.9)))
        assert mid[0] <= 1.5 * mid[1] and high[0] <= 2.0 * high[1], (
            f"{what}: row errors' median {mid[0]:.3e} and ninth decile {high[0]:.3e}; rounding alone moves the plain model "
            f"by {mid[1]:.3e} and {high[1]:.3e}; |logits| {self.scale:.3e}; {len(self.err)} rows")  # fmt: skip


def reference(raw, weights, ids, refs, key, dtype):
    if key not in refs:
        refs[key] = (plain.logits(raw, weights, ids), plain.logits(raw, weights, ids, rounded=True) if dtype == "bfloat16" else None)
    return refs[key]


def compare(replay, steps, requests, raw, weights, refs, dtype):
    at = {rid: 0 for rid in requests}
    result = Against()
    for s in steps:
        logits = replay.step(s["entries"], s["end"])
        k = 0
        for e in s["entries"]:
            rid = e["id"]
            exact, rounded = reference(raw, weights, requests[rid], refs, rid, dtype)
            for w in e["want"]:
                place = at[rid] + w
                result.add(logits[k], exact[place], None if rounded is None else rounded[place])
                k += 1
            at[rid] += len(e["tokens"])
    return result


# ---- whole models -------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_whole_decoded_in_portions_and_mixed(case, dtype):
    """One model, several ways of cutting the same requests: all must give the plain model's logits at every place.
    Every way starts on pages and state slots that the way before used."""
    raw = CASES[case]
    weights = random_weights(raw, seed=len(case))
    vocab = raw["vocab"]
    requests = {"a": rc.random_ids(vocab, 71, 1), "b": rc.random_ids(vocab, 37, 2), "c": rc.random_ids(vocab, 2, 3),
                "d": rc.random_ids(vocab, 1, 4), "e": rc.random_ids(vocab, 50, 5)}  # fmt: skip
    refs = {}
    replay = make_replay(raw, weights, dtype, max_tokens=4 * 128)
    manager = replay.manager
    free_pages = manager.num_free
    ways = [(rid + " whole", rc.whole(rid, ids)) for rid, ids in requests.items()]
    ways.append(("a decoded", rc.prefill_then_decode("a", requests["a"], tail=40)))
    ways.append(("b token by token", rc.prefill_then_decode("b", requests["b"], tail=36)))
    ways.append(("a portions", rc.portions("a", requests["a"])))
    ways.append(("e portions of two", rc.portions("e", requests["e"], sizes=(2,))))
    ways.append(("mixed", rc.mixed(requests, seed=7, max_live=3)))
    ways.append(("mixed again", rc.mixed(requests, seed=8, max_live=4, sizes=(2, 3, 16, 17, 5))))
    total = Against()
    for name, steps in ways:
        result = compare(replay, steps, requests, raw, weights, refs, dtype)
        if dtype == "float32":
            result.check(dtype, f"{case} {name}")
        total.take(result)
        assert manager.num_free == free_pages, name
    total.check(dtype, case)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [4, 8, 64])
def test_pages_of_other_sizes(block_size, dtype):
    raw = CASES["latent_first"]
    weights = random_weights(raw, seed=9)
    requests = {"a": rc.random_ids(raw["vocab"], 90, 6), "b": rc.random_ids(raw["vocab"], 33, 7), "c": rc.random_ids(raw["vocab"], 70, 8)}
    replay = make_replay(raw, weights, dtype, max_tokens=3 * 128, block_size=block_size, max_live=3)
    refs, total = {}, Against()
    for steps in (rc.portions("a", requests["a"], sizes=(5, 2, 30, 3, 9)), rc.mixed(requests, seed=3, max_live=3),
                  rc.prefill_then_decode("c", requests["c"], tail=45)):  # fmt: skip
        total.take(compare(replay, steps, requests, raw, weights, refs, dtype))
    total.check(dtype, f"pages of {block_size}")
    assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_many_pages(dtype):
    """A short prompt and 150 tokens decoded one by one (captured steps) over pages of 8 tokens; a second request
    starts beside it later, decodes from another position and ends first."""
    raw = CASES["latents"] if dtype == "bfloat16" else CASES["latent_first"]
    weights = random_weights(raw, seed=21)
    a, b = rc.random_ids(raw["vocab"], 160, 11), rc.random_ids(raw["vocab"], 90, 12)
    refs = {}
    replay = make_replay(raw, weights, dtype, max_tokens=320, block_size=8 if dtype == "float32" else 16)
    got = {"a": [replay.step([{"id": "a", "tokens": a[:10], "want": list(range(10))}], [])], "b": []}
    for i in range(10, 160):
        entries = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        j = i - 40
        if j == 0:
            entries.append({"id": "b", "tokens": b[:3], "want": [0, 1, 2]})
        elif 3 <= j < 90:
            entries.append({"id": "b", "tokens": [b[j]], "want": [0]})
        out = replay.step(entries, [e["id"] for e in entries if (e["id"] == "a" and i == 159) or (e["id"] == "b" and j == 89)])
        got["a"].append(out[:1])
        if len(entries) > 1:
            got["b"].append(out[1:])
    for rid, ids in (("a", a), ("b", b)):
        result = Against()
        result.add(torch.cat(got[rid]), *reference(raw, weights, ids, refs, rid, dtype))
        result.check(dtype, rid)
    assert replay.manager.num_free == replay.manager.num_blocks
    if dtype == "float32":
        assert replay.runner.decode_graphs.graphs, "decode steps were not captured"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype):
    """The engine's own entry point: prompts of unequal lengths under a small token budget (so prompts are cut) and a
    pool small enough that pages and slots are used again; greedy tokens are the plain model's."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    raw = CASES["latent_first"]
    weights = random_weights(raw, seed=33)
    model = build_model(raw, weights, dtype)
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=24, max_model_len=128, max_num_seqs=2,
                                               max_num_batched_tokens=12))  # fmt: skip
    assert not engine.scheduler.manager.prefix_reuse_possible
    prompts = [rc.random_ids(raw["vocab"], n, 40 + n) for n in (5, 29, 1, 14)]
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True))
    assert engine.scheduler.manager.num_free == 24
    replay = make_replay(raw, weights, dtype, max_tokens=128) if dtype == "bfloat16" else None
    for n, (prompt, out) in enumerate(zip(prompts, outs)):
        assert len(out) == 7
        seq = list(prompt)
        for t in out:
            if dtype == "float32":
                assert t == int(plain.logits(raw, weights, seq)[-1].argmax())
            else:
                ref = replay.step([{"id": f"r{n}", "tokens": seq, "want": [len(seq) - 1]}], [f"r{n}"])[0]
                assert ref[t] >= ref.max() - 2e-2 * max(1.0, float(ref.abs().max()))
            seq.append(t)


def test_the_replay_tool_on_a_folder(tmp_path):
    """The replay tool's own main on a model folder written here: config.json names the architecture."""
    import io

    import numpy as np
    from safetensors.torch import save_file

    from atomserve_amd.engine import replay

    raw = CASES["wide_keys"]
    weights = random_weights(raw, seed=17)
    folder = tmp_path / "model"
    os.makedirs(folder)
    save_file({k: v.bfloat16().contiguous() for k, v in weights.items()}, str(folder / "model.safetensors"))
    (folder / "config.json").write_text(json.dumps(raw))
    ids = rc.random_ids(raw["vocab"], 30, 2)
    lines = [json.dumps({"step": 0, "entries": [{"id": "x", "tokens": ids[:21], "want": [3, 20]}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "x", "tokens": ids[21:], "want": [8]}], "end": ["x"]})]  # fmt: skip
    out = tmp_path / "out"
    assert replay.main(["--model", str(folder), "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                       stdin=io.StringIO("\n".join(lines) + "\n")) == 0  # fmt: skip
    ref = plain.logits(raw, weights, ids)
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    assert (got0 - ref[[3, 20]]).abs().max() <= 3e-5 * float(ref.abs().max())
    assert (got1 - ref[[29]]).abs().max() <= 3e-5 * float(ref.abs().max())


def test_the_command_line_generates_from_a_folder_and_from_random_weights(tmp_path, capsys):
    from safetensors.torch import save_file

    from atomserve_amd.engine import cli

    raw = CASES["latent_first"]
    weights = random_weights(raw, seed=17)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    save_file({k: v.bfloat16().contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    prompt = rc.random_ids(raw["vocab"], 21, 3)
    common = ["--dtype", "fp32", "--prompt-ids", " ".join(map(str, prompt)), "--max-tokens", "5", "--temperature", "0",
              "--ignore-eos", "--kv-mem-gb", "0.05", "--max-num-seqs", "2", "--max-batched-tokens", "16"]  # fmt: skip
    assert cli.main([str(tmp_path), *common]) == 0
    lines = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    want, seq = [], list(prompt)
    for _ in range(5):
        want.append(int(plain.logits(raw, weights, seq)[-1].argmax()))
        seq.append(want[-1])
    assert lines[-1]["output_ids"] == want
    assert cli.main([str(tmp_path), "--random-weights", "3", *common]) == 0
    lines = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert len(lines[-1]["output_ids"]) == 5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_stream_after_every_layer(dtype):
    """The stream after every layer (after the average over the layers' results) against the plain model's: a fault
    shows at the first layer it touches."""
    raw = CASES["latent_first"]
    weights = random_weights(raw, seed=4)
    ids = rc.random_ids(raw["vocab"], 45, 3)
    want, rounded = [], []
    plain.forward(raw, weights, ids, layers_out=want)
    if dtype == "bfloat16":
        plain.forward(raw, weights, ids, bf16=True, layers_out=rounded)
    replay = make_replay(raw, weights, dtype, max_tokens=64)
    seen = []
    for block in replay.model.blocks:
        inner = block.forward

        def watched(x, *a, inner=inner, **k):
            d = inner(x, *a, **k)
            assert d is None
            seen.append(x.clone().cpu())
            return d

        block.forward = watched
    replay.step([{"id": "a", "tokens": ids, "want": [44]}], ["a"])
    assert len(seen) == len(want) == len(raw["layers"])
    for i, (got, ref) in enumerate(zip(seen, want)):
        rows = (got.double() - ref).abs().max(-1).values
        if dtype == "float32":
            assert float(rows.max()) <= 2e-5 * float(ref.abs().max()), f"layer {i}: {float(rows.max()):.3e} of {float(ref.abs().max()):.3e}"
            continue
        # bfloat16: against what rounding the stored activations moves the plain model's own stream after this layer, as
        # distributions (a token whose router logits lie within rounding of each other may take another expert)
        noise = (rounded[i] - ref).abs().max(-1).values
        assert float(rows.median()) <= 2.0 * float(noise.median()) and float(rows.quantile(0.9)) <= 2.0 * float(noise.quantile(0.9)), (
            f"layer {i}: rows' median {float(rows.median()):.3e} and ninth decile {float(rows.quantile(0.9)):.3e}; the plain "
            f"model's {float(noise.median()):.3e} and {float(noise.quantile(0.9)):.3e}")  # fmt: skip


# ---- each mechanism alone -------------------------------------------------------------------------------------


def bf(x):
    return x.bfloat16().float()


def dev(t, dtype=None):
    return t.to(DEV).to(dtype if dtype is not None else t.dtype).contiguous()


def step_rows(cuts, starts, slots):
    """The tensors that kernels with per-request state take for rows of `cuts` tokens laid one after another."""
    first = [sum(cuts[:i]) for i in range(len(cuts))]
    tok_row = [r for r, n in enumerate(cuts) for _ in range(n)]
    mk = lambda v: torch.tensor(v, dtype=I32, device=DEV)  # noqa: E731
    return mk(tok_row), mk(first), mk(cuts), mk(starts), mk(slots)


def in_pieces(T, cuts):
    at = 0
    for n in cuts:
        yield at, n
        at += n
    assert at == T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(96, 1), (96, 3), (40, 5), (2048, 2), (264, 4)])
def test_grouped_norm_and_token_shift(sizes, dtype):
    """The norm in groups, and the shift across the cuts of a request that comes in rows beside another request's rows:
    the row before a cut waits in the request's slot, which held another request's row before."""
    from atomserve_amd.kernels import ops

    n, groups = sizes
    gen = torch.Generator().manual_seed(n + groups)
    T = 23
    x = {r: torch.randn(T, n, generator=gen) * 3 for r in "ab"}
    gain, mu = bf(1 + 0.1 * torch.randn(n, generator=gen)), bf(torch.rand(n, generator=gen))
    want = {r: plain.token_shift(plain.grouped_rms_norm(x[r].double(), gain.double(), 1e-5, groups), mu.double()) for r in "ab"}
    tol = 3e-6 if dtype == "float32" else 1e-2
    out = torch.empty((T, n), dtype=DTYPES[dtype], device=DEV)
    ops.group_norm(dev(x["a"]), dev(gain), 1e-5, groups, out)
    plain_norm = plain.grouped_rms_norm(x["a"].double(), gain.double(), 1e-5, groups)
    assert (out.float().cpu() - plain_norm).abs().max() <= tol * float(plain_norm.abs().max())
    state = torch.full((3, n), 7.0, device=DEV)  # what earlier requests left
    got = {r: [] for r in "ab"}
    pieces = {"a": list(in_pieces(T, [1, 2, 9, 1, 1, 7, 2])), "b": list(in_pieces(T, [5, 1, 1, 2, 12, 1, 1]))}
    for (a0, an), (b0, bn) in zip(pieces["a"], pieces["b"]):
        xs = torch.cat([x["b"][b0 : b0 + bn], x["a"][a0 : a0 + an]])
        o = torch.empty((an + bn, n), dtype=DTYPES[dtype], device=DEV)
        ops.group_norm_shift(dev(xs), dev(gain), dev(mu), 1e-5, groups, step_rows([bn, an], [b0, a0], [2, 0]), state, o)
        got["b"].append(o[:bn].float().cpu())
        got["a"].append(o[bn:].float().cpu())
    for r in "ab":
        assert (torch.cat(got[r]) - want[r]).abs().max() <= tol * float(want[r].abs().max()), r
    # a row that does not write leaves the slot as it was
    before = state.clone()
    ops.group_norm_shift(dev(x["a"][:4]), dev(gain), dev(mu), 1e-5, groups, step_rows([4], [0], [1]), state,
                         torch.empty((4, n), dtype=DTYPES[dtype], device=DEV), writes=False)  # fmt: skip
    assert torch.equal(state, before)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_average_over_the_layers_results(dtype):
    from atomserve_amd.kernels import ops

    T, w, slots = 9, 72, 5
    gen = torch.Generator().manual_seed(5)
    kept = torch.zeros((slots, T, w), device=DEV)
    results = [torch.randn(T, w, generator=gen) for _ in range(slots)]
    kept[0].copy_(results[0])
    x = dev(results[0])
    for n in range(1, slots):
        coef = torch.randn(n + 1, generator=gen)
        delta = bf(results[n] - x.cpu())  # the layer's result is the stream plus what its last part left pending
        before = x.cpu().double()
        ops.depth_average(x, dev(delta, DTYPES[dtype]), kept, dev(coef), n)
        full = before + delta.double()
        assert (kept[n].cpu().double() - full).abs().max() <= 1e-6 * float(full.abs().max())
        want = sum(coef[j].double() * kept[j].cpu().double() for j in range(n + 1))
        assert (x.cpu().double() - want).abs().max() <= 3e-6 * max(1.0, float(want.abs().max()))
    y = dev(results[1])
    ops.depth_average(y, None, kept, dev(torch.tensor([0.25, -2.0])), 1)  # nothing pending: the stream is the result
    assert (y.cpu() - (0.25 * results[0] - 2.0 * results[1])).abs().max() <= 1e-5


def run_decay(q, k, v, decay, act, k_scale, cuts, dtype, slot=1, state=None, kernel=None):
    """The scan over one request cut into rows of `cuts` tokens (one call each), q, k, v given before the activation.
    kernel: "decay_scan", "decay_chunks" or (single tokens) "decay_step" to name one; None: as a step would choose (single tokens as a decode step)."""
    from atomserve_amd.kernels import ops

    T, H, D = q.shape
    E = v.shape[2]
    proj = dev(torch.cat([torch.zeros(T, 3), q.reshape(T, -1), v.reshape(T, -1), k.reshape(T, -1)], 1), DTYPES[dtype])
    q_off, v_off, k_off = 3, 3 + H * D, 3 + H * D + H * E
    if state is None:
        state = torch.full((3, H, D, E), 5.0, device=DEV)
    outs = []
    for at, n in in_pieces(T, cuts):
        o = torch.empty((n, H, E), dtype=torch.float32, device=DEV)
        rows = step_rows([n], [at], [slot])
        if kernel is None and n == 1:
            rows = (None, *rows[1:])
        getattr(ops, kernel or "decay_attention")(proj[at : at + n].contiguous(), q_off, k_off, v_off, H, D, E, act, k_scale,
                                                  dev(torch.tensor(decay)), state, rows, o)  # fmt: skip
        outs.append(o.cpu())
    return torch.cat(outs), state


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(2, 16, 16), (3, 8, 40), (1, 72, 24), (5, 33, 7), (2, 128, 64), (1, 200, 130)])
def test_linear_attention_with_decays(shape, dtype):
    """S = decay S + k v^T, o = S^T q against the plain scan: both flavours (silu on q, k, v; a factor on k), keys
    narrower and wider than values and than a lane's slice, whole, token by token and in rows; the slot starts full of
    another request's numbers."""
    H, D, E = shape
    T = 67
    gen = torch.Generator().manual_seed(sum(shape))
    q, k, v = bf(torch.randn(T, H, D, generator=gen)), bf(torch.randn(T, H, D, generator=gen)), bf(torch.randn(T, H, E, generator=gen))
    decay = [1.0, 0.5, 0.99, 0.9375, 0.0][:H]
    silu = torch.nn.functional.silu
    for act, k_scale in (("silu", 1.0), (None, D**-0.5)):
        f = (lambda t: silu(t.double())) if act else (lambda t: t.double())
        want = plain.decayed_state_scan(f(q), f(k) * k_scale, f(v), decay).float()
        tol = 2e-5 * float(want.abs().max())
        kernels = ("decay_scan", "decay_chunks") if D <= 128 else ("decay_scan",)
        ways = [(c, kn) for c in ([T], [1] * T, [2, 31, 1, 1, 30, 2], [32, 33, 2]) for kn in kernels] + [([1] * T, None), ([T], None)]
        if D <= 128 and E % 4 == 0:
            ways.append(([1] * T, "decay_step"))
        for cuts, kernel in ways:
            got, state = run_decay(q, k, v, decay, act, k_scale, cuts, dtype, kernel=kernel)
            assert (got - want).abs().max() <= tol, f"{shape} {act} {cuts} {kernel}: {float((got - want).abs().max()):.3e} of {float(want.abs().max()):.3e}"
        assert bool((state[0] == 5.0).all()) and bool((state[2] == 5.0).all())  # the other slots are not touched


def test_linear_attention_keeps_a_far_key_and_forgets_by_its_decay():
    """All keys are zero but one, 300 tokens back: what a query reads of it later is decay^distance (q . k) v exactly,
    whatever the rows' cuts (also one right behind the key, and one right before it)."""
    H, D, E, T, special = 2, 24, 8, 420, 100
    gen = torch.Generator().manual_seed(0)
    q = bf(torch.randn(T, H, D, generator=gen))
    k, v = torch.zeros(T, H, D), bf(torch.randn(T, H, E, generator=gen))
    k[special] = bf(torch.randn(H, D, generator=gen))
    decay = [1.0, 0.96875]
    ways = ([T], [special, T - special], [special + 1, T - special - 1], [special, 1, 1, 2, T - special - 4], [64] * 6 + [36])
    for cuts, kernel in [(c, kn) for c in ways for kn in ("decay_scan", "decay_chunks")]:
        got, _ = run_decay(q, k, v, decay, None, 1.0, cuts, "float32", kernel=kernel)
        assert bool((got[:special] == 0).all())
        for t in (special, special + 1, special + 64, T - 1):
            for h in range(H):
                want = decay[h] ** (t - special) * float(q[t, h] @ k[special, h]) * v[special, h]
                assert (got[t, h] - want).abs().max() <= 1e-5 * max(1.0, float(want.abs().max())), (cuts, kernel, t, h)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(3, 40, 5), (3, 40, 8), (2, 7, 4), (32, 128, 64)])
def test_linear_attention_output_norm_and_gate(sizes, dtype):
    """Rows and groups that start on 16 bytes (four values a load) and others."""
    from atomserve_amd.kernels import ops

    T, (H, E, off) = 11, sizes
    gen = torch.Generator().manual_seed(2)
    o = torch.randn(T, H, E, generator=gen) * 4
    proj = bf(torch.randn(T, off + H * E, generator=gen))
    gain = bf(1 + 0.1 * torch.randn(H * E, generator=gen))
    tol = 3e-6 if dtype == "float32" else 1e-2
    out = torch.empty((T, H * E), dtype=DTYPES[dtype], device=DEV)
    ops.decay_finish(dev(o).view(T, H * E), H, 1e-5, None, dev(proj, DTYPES[dtype]), off, "silu", out)
    want = plain.rms(o.double(), 1e-5).reshape(T, -1) * torch.nn.functional.silu(proj[:, off:].double())
    assert (out.float().cpu() - want).abs().max() <= tol * float(want.abs().max())
    ops.decay_finish(dev(o).view(T, H * E), 1, 1e-5, dev(gain), dev(proj, DTYPES[dtype]), off, "sigmoid", out)
    want = plain.rms(o.double().reshape(T, -1), 1e-5) * gain.double() * torch.sigmoid(proj[:, off:].double())
    assert (out.float().cpu() - want).abs().max() <= tol * float(want.abs().max())


def test_scaled_rotation_table():
    """Cosines and sines of the stretched rotation at positions up to 100,000 against the plain formula."""
    from atomserve_amd.parts.base import BuildEnv, build
    from atomserve_amd.parts.plan import RotarySpec, ScaledRotarySpec

    class Step:
        shared = {}
        positions = torch.tensor([0, 1, 2, 63, 64, 511, 512, 4095, 100000], dtype=I32, device=DEV)
        num_tokens = 9

    env = BuildEnv(torch.float32, torch.device(DEV))
    for dims, base, scaling in ((16, 200000.0, (6.0, 256, 24.0, 1.5)), (6, 50.0, (3.0, 20, 4.0, 0.5)), (64, 10000.0, (40.0, 4096, 16.0, 2.0)),
                                (2, 7.0, (2.0, 16, 4.0, 0.5)), (8, 100.0, None)):  # fmt: skip
        rot = {"dims": dims, "base": base}
        if scaling:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        spec = ScaledRotarySpec("rope_half_scaled", dims, base, *scaling) if scaling else RotarySpec("rope_half", dims, base)
        Step.shared = {}
        table = build("position", spec, env).prepare(Step).cpu().double()
        cos, sin = plain.yarn_angles(Step.positions.cpu(), rot)
        assert (table[..., 0] - cos).abs().max() <= 2e-6 * (1 + 0.1 * math.log(scaling[0]) if scaling else 1.0)
        assert (table[..., 1] - sin).abs().max() <= 2e-6 * (1 + 0.1 * math.log(scaling[0]) if scaling else 1.0)


def latent_pages(c, kr, bs, width, gen, dtype, junk):
    """The latent and the shared key part of one sequence as the cache holds them, in pages handed out in a random
    order among others full of `junk`."""
    L, rank = c.shape
    n = -(-L // bs)
    pool = 2 * n + 3
    order = torch.randperm(pool, generator=gen)[:n]
    kp = torch.full((pool, 1, bs, width), junk)
    vp = torch.full((pool, 1, width, bs), junk)
    row = torch.zeros(L, width)
    row[:, :rank] = c
    row[:, rank : rank + kr.shape[1]] = kr
    val = torch.zeros(L, width)
    val[:, :rank] = c
    for j in range(L):
        kp[order[j // bs], 0, j % bs] = row[j]
        vp[order[j // bs], 0, :, j % bs] = val[j]
    return dev(kp, DTYPES[dtype]), dev(vp, DTYPES[dtype]), order.to(I32).view(1, n).to(DEV)


def latent_attend(q, c, kr, uk, uv, scale, dtype, bs, gen, singles=True):
    """Queries [L, H, D + R] (turned already) over the cached latent, through the kernels: absorbed queries, the
    paged attention over one kv head, values expanded.  Returns [L, H, E]."""
    from atomserve_amd.kernels import ops

    L, H, DR = q.shape
    rank, R = c.shape[1], kr.shape[1]
    D, E = DR - R, uv.shape[0] // H
    t = DTYPES[dtype]
    width = -(-(rank + R) // 32) * 32
    kp, vp, table = latent_pages(c, kr, bs, width, gen, dtype, junk=3.0)
    ones = torch.zeros(L, max(R // 2, 1), 2)
    ones[..., 0] = 1.0  # cos 1, sin 0: the queries come turned
    qa = torch.empty((L, H, width), dtype=t, device=DEV)
    uk_t = dev(uk.view(H, D, rank).transpose(1, 2), t)  # with it, bfloat16 prompts multiply on the matrix cores
    ops.latent_q_absorb(dev(q.reshape(L, -1), t), dev(uk, t), H, D, R, rank, dev(ones) if R else None, qa, uk_t=uk_t)
    few = torch.empty((5, H, width), dtype=t, device=DEV)  # and few tokens through the general kernel: the same
    ops.latent_q_absorb(dev(q.reshape(L, -1)[40:45], t), dev(uk, t), H, D, R, rank, dev(ones[40:45]) if R else None, few, uk_t=uk_t)
    assert (few.float() - qa[40:45].float()).abs().max() <= (1e-5 if dtype == "float32" else 2e-2) * float(qa.float().abs().max())
    heads = torch.zeros((L, H, width), dtype=t, device=DEV)
    positions = torch.arange(L, dtype=I32, device=DEV)
    rows = torch.zeros(L, dtype=I32, device=DEV)
    if singles or not ops.attn_prefill_supported(t, width, bs):
        ops.attn_single_query(qa, kp, vp, None, positions, rows, table, heads, scale, 0, L)
    else:
        tiles = torch.tensor([(f, min(64, L - f), 0, f) for f in range(0, L, 64)], dtype=I32, device=DEV)
        ops.attn_prefill(qa, kp, vp, tiles, table, heads, scale, 0, L)
    out = torch.empty((L, H * E), dtype=t, device=DEV)
    uv_t = dev(uv.view(H, E, rank).transpose(1, 2), t)
    ops.latent_v_expand(heads, uv_t, rank, None, 0, out, uv=dev(uv, t))
    gate = bf(torch.randn(7, 3 + H * E, generator=gen))
    gated = torch.empty((7, H * E), dtype=t, device=DEV)
    ops.latent_v_expand(heads[50:57].contiguous(), uv_t, rank, dev(gate, t), 3, gated, uv=dev(uv, t))
    want = out[50:57].float().cpu() * torch.sigmoid(gate[:, 3:])
    assert (gated.float().cpu() - want).abs().max() <= (1e-5 if dtype == "float32" else 2e-2) * float(want.abs().max())
    return out.float().cpu().view(L, H, E)


def plain_latent_attention(q, c, kr, uk, uv, scale):
    L, H, DR = q.shape
    R = kr.shape[1]
    D = DR - R
    k = (c @ uk.t()).view(L, H, D)
    v = (c @ uv.t()).view(L, H, -1)
    s = torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihr,jr->hij", q[..., D:], kr)
    s = (s * scale).masked_fill(~torch.ones(L, L, dtype=torch.bool).tril(), float("-inf"))
    return torch.einsum("hij,jhe->ihe", torch.softmax(s, -1), v)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 8, 8, 16, 40), (18, 4, 4, 8, 24), (4, 32, 32, 32, 128), (2, 40, 0, 16, 64), (6, 16, 2, 8, 222),
                                   (32, 24, 64, 16, 192), (48, 8, 16, 8, 80), (8, 64, 32, 40, 96)])
def test_attention_through_a_latent(shape, dtype):
    """Random queries, latents and key parts: heads' keys and values written out from the latent in the plain form,
    absorbed into the queries and applied after the attention in the kernels; as single tokens and in tiles."""
    H, D, R, E, rank = shape
    L, gen = 150, torch.Generator().manual_seed(sum(shape))
    q, c, kr = bf(torch.randn(L, H, D + R, generator=gen)), bf(torch.randn(L, rank, generator=gen)), bf(torch.randn(L, R, generator=gen))
    uk, uv = bf(0.3 * torch.randn(H * D, rank, generator=gen)), bf(0.3 * torch.randn(H * E, rank, generator=gen))
    want = plain_latent_attention(q.double(), c.double(), kr.double(), uk.double(), uv.double(), 0.2).float()
    tol = (3e-5 if dtype == "float32" else 3e-2) * float(want.abs().max())
    for bs, singles in ((16, True), (16, False), (4, True), (64, False)):
        got = latent_attend(q, c, kr, uk, uv, 0.2, dtype, bs, gen, singles)
        assert (got - want).abs().max() <= tol, f"{shape} pages of {bs}: {float((got - want).abs().max()):.3e} of {float(want.abs().max()):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 8, 8, 16, 300, 16), (2, 24, 2, 8, 514, 4), (5, 8, 4, 8, 40, 64)])
def test_attention_over_a_wide_latent(shape, dtype):
    """The kernel for pages wider than the paged attention kernels' heads (and any narrower ones) against the plain
    form: 600 positions (three blocks of keys), a far latent that every query matches from position 280 on."""
    from atomserve_amd.kernels import ops

    H, D, R, E, rank, bs = shape
    L, gen = 600, torch.Generator().manual_seed(sum(shape))
    t = DTYPES[dtype]
    q, c, kr = bf(torch.randn(L, H, D + R, generator=gen)), bf(torch.randn(L, rank, generator=gen)), bf(torch.randn(L, R, generator=gen))
    uk, uv = bf(0.3 * torch.randn(H * D, rank, generator=gen)), bf(0.3 * torch.randn(H * E, rank, generator=gen))
    c[280] *= 3.0
    want = plain_latent_attention(q.double(), c.double(), kr.double(), uk.double(), uv.double(), 0.05).float()
    width = -(-(rank + R) // 8) * 8
    kp, vp, table = latent_pages(c, kr, bs, width, gen, dtype, junk=3.0)
    ones = torch.zeros(L, R // 2, 2)
    ones[..., 0] = 1.0
    qa = torch.empty((L, H, width), dtype=t, device=DEV)
    ops.latent_q_absorb(dev(q.reshape(L, -1), t), dev(uk, t), H, D, R, rank, dev(ones), qa)
    heads = torch.zeros((L, H, width), dtype=t, device=DEV)
    ops.wide_attend(qa, kp, vp, torch.arange(L, dtype=I32, device=DEV), torch.zeros(L, dtype=I32, device=DEV), table, heads, 0.05, L)
    out = torch.empty((L, H * E), dtype=t, device=DEV)
    ops.latent_v_expand(heads, dev(uv.view(H, E, rank).transpose(1, 2), t), rank, None, 0, out)
    got = out.float().cpu().view(L, H, E)
    tol = (3e-5 if dtype == "float32" else 3e-2) * float(want.abs().max())
    assert (got - want).abs().max() <= tol, f"{shape}: {float((got - want).abs().max()):.3e} of {float(want.abs().max()):.3e}"


@pytest.mark.parametrize("block_size", [8, 16, 64])
def test_a_far_latent_and_pages_borders_show(block_size):
    """One cached latent that every head's query matches far better than any other: from its position on every
    output is that latent's value, before it the others'.  It stands at the first position, at a page's border on
    either side, and hundreds of tokens back."""
    H, D, R, E, rank, L = 3, 8, 4, 6, 28, 700
    gen = torch.Generator().manual_seed(block_size)
    uk, uv = bf(torch.randn(H * D, rank, generator=gen)), bf(torch.randn(H * E, rank, generator=gen))
    unit = torch.zeros(rank)
    unit[5] = 1.0
    for special in (0, block_size - 1, block_size, 333, 2 * block_size + 1):
        c = bf(0.05 * torch.randn(L, rank, generator=gen))
        c[special] = 8.0 * unit
        kr = bf(0.05 * torch.randn(L, R, generator=gen))
        q = torch.zeros(L, H, D + R)
        q[:, :, :D] = bf(8.0 * uk[:, 5].view(H, D) / uk[:, 5].view(H, D).pow(2).sum(-1, keepdim=True))  # U_h^T q_h . unit = 8
        want = plain_latent_attention(q.double(), c.double(), kr.double(), uk.double(), uv.double(), 1.0).float()
        value = (8.0 * uv[:, 5]).view(H, E)
        assert (want[special:] - value).abs().max() <= 1e-2 and (special == 0 or float(want[:special].abs().max()) < 0.5 * float(value.abs().max()))
        for singles in (True, False):
            got = latent_attend(q, c, kr, uk, uv, 1.0, "float32", block_size, gen, singles)
            assert (got - want).abs().max() <= 1e-4 * float(value.abs().max()), f"latent at {special}, pages of {block_size}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_latent_is_stored_normed_and_the_key_part_turned(dtype):
    from atomserve_amd.kernels import ops

    T, rank, R, bs, width = 21, 40, 8, 8, 64
    gen = torch.Generator().manual_seed(8)
    proj = bf(torch.randn(T, 7 + rank + R + 5, generator=gen))
    gain = bf(1 + 0.1 * torch.randn(rank, generator=gen))
    positions = torch.arange(100, 100 + T)
    rot = {"dims": R, "base": 50.0}
    cos, sin = plain.yarn_angles(positions, rot)
    table = torch.stack([cos, sin], -1).float()
    slots = torch.randperm(6 * bs, generator=gen)[:T].to(I32)
    slots[4] = -1
    t = DTYPES[dtype]
    kp = torch.full((6, 1, bs, width), 9.0, dtype=t, device=DEV)
    vp = torch.full((6, 1, width, bs), 9.0, dtype=t, device=DEV)
    ops.latent_kv_store(dev(proj, t), 7, rank, R, dev(gain), 1e-5, dev(table), dev(slots), kp, vp)
    c = plain.rms(proj[:, 7 : 7 + rank].double(), 1e-5) * gain.double()
    kr = plain.rotate_half(proj[:, 7 + rank : 7 + rank + R].double(), cos, sin)
    tol = 1e-5 if dtype == "float32" else 2e-2
    for i in range(T):
        if slots[i] < 0:
            continue
        page, off = int(slots[i]) // bs, int(slots[i]) % bs
        key, value = kp[page, 0, off].float().cpu().double(), vp[page, 0, :, off].float().cpu().double()
        assert (key[:rank] - c[i]).abs().max() <= tol * float(c.abs().max()) and (key[rank : rank + R] - kr[i]).abs().max() <= tol * float(kr.abs().max())
        assert bool((key[rank + R :] == 0).all()) and torch.equal(value[:rank], key[:rank]) and bool((value[rank:] == 0).all())
    assert int((kp.float() == 9.0).sum()) == (6 * bs - (T - 1)) * width  # nothing else was written


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("limit", [0.5, 7.0])
def test_gated_activation_with_limits(limit, dtype):
    from atomserve_amd.kernels import ops

    gen = torch.Generator().manual_seed(1)
    gate_up = bf(torch.randn(13, 2 * 44, generator=gen) * 3)
    out = torch.empty((13, 44), dtype=DTYPES[dtype], device=DEV)
    ops.clamped_gate(dev(gate_up, DTYPES[dtype]), out, limit)
    want = plain.clamped_gate(gate_up[:, :44].double(), gate_up[:, 44:].double(), limit)
    assert (out.float().cpu() - want).abs().max() <= (2e-6 if dtype == "float32" else 1e-2) * float(want.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 8, 24, 70])
def test_gated_product_with_limits(rows, dtype):
    """The product [gate | up] with the activation: few bfloat16 rows through the kernel that applies it on its way
    out, the others through the product and the activation's own kernel; both round the two products first."""
    from atomserve_amd.kernels import ops

    K, inner, limit = 256, 96, 1.25
    gen = torch.Generator().manual_seed(rows)
    a, w = bf(torch.randn(rows, K, generator=gen)), bf(0.2 * torch.randn(2 * inner, K, generator=gen))
    t = DTYPES[dtype]
    out = torch.empty((rows, inner), dtype=t, device=DEV)
    for weights in (dev(w, t), ops.Streamed(dev(w, t), True)):
        ops.gemm_clamped_gate(dev(a, t), weights, out, limit, ops.ProductChoices(fixed=True))
        prod = a.double() @ w.double().t()
        if dtype == "bfloat16":
            prod = bf(prod.float()).double()
        want = plain.clamped_gate(prod[:, :inner], prod[:, inner:], limit)
        assert (out.float().cpu() - want).abs().max() <= (3e-6 if dtype == "float32" else 1e-2) * float(want.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(5, 2, 40, 24), (7, 1, 24, 0), (3, 3, 16, 16), (70, 9, 8, 8), (2, 2, 264, 0)])
def test_gated_routed_experts_alone(sizes, dtype):
    """The router's choice (logits with a bias, the largest) and weights (softmax over the chosen) against the plain
    ones, the experts' weighted sum and the shared expert; a token alone gives what it gives in company."""
    from atomserve_amd.kernels import ops
    from atomserve_amd.parts.base import BuildEnv, build
    from atomserve_amd.parts.plan import GatedRoutedExpertsSpec

    experts, top, ff, shared = sizes
    hidden, T = 72, 41
    gen = torch.Generator().manual_seed(sum(sizes))
    mat = lambda *s, sd=0.2: bf(sd * torch.randn(*s, generator=gen))  # noqa: E731
    w = {"x.router": mat(experts, hidden, sd=0.5), "x.router.b": mat(experts, sd=1.0)}
    for e in range(experts):
        w[f"x.e{e}.gate"], w[f"x.e{e}.up"], w[f"x.e{e}.down"] = mat(ff, hidden, sd=0.4), mat(ff, hidden, sd=0.4), mat(hidden, ff)
    f = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": 1.25}}
    if shared:
        w["x.shared.gate"], w["x.shared.up"], w["x.shared.down"] = mat(shared, hidden, sd=0.4), mat(shared, hidden, sd=0.4), mat(hidden, shared)
        f["shared"] = {"ff": shared, "limit": 0.75}
    env = BuildEnv(DTYPES[dtype], torch.device(DEV), products=ops.ProductChoices(fixed=True))
    part = build("feed_forward", GatedRoutedExpertsSpec("gated_routed_experts", hidden, ff, experts, top, "clamped_swish", 1.25,
                                                        shared_size=shared, shared_limit=0.75), env)  # fmt: skip
    t = {"router.weight": w["x.router"], "router.bias": w["x.router.b"],
         "gate.weight": torch.stack([w[f"x.e{e}.gate"] for e in range(experts)]),
         "up.weight": torch.stack([w[f"x.e{e}.up"] for e in range(experts)]),
         "down.weight": torch.stack([w[f"x.e{e}.down"] for e in range(experts)])}  # fmt: skip
    if shared:
        t["shared_gate_up.weight"] = torch.cat([w["x.shared.gate"], w["x.shared.up"]])
        t["shared_down.weight"] = w["x.shared.down"]
    part.bind({k: dev(v, DTYPES[dtype]) for k, v in t.items()})
    h = bf(torch.randn(T, hidden, generator=gen))
    hd = dev(h, DTYPES[dtype])
    wd = {k: v.double() for k, v in w.items()}

    class Step:
        shared = {}

    route = ops.moe_route_scores(hd, part.router_weight, top, "softmax_of_chosen", part.router_bias)
    torch.cuda.synchronize()
    chosen, weights, z = plain.route(h.double(), wd, "x.", top)
    pairs = torch.zeros(T * top, dtype=torch.int64)
    order, tiles, n_tiles = route.order.cpu(), route.tiles.cpu(), int(route.counts.cpu())
    for e, first, count in tiles[:n_tiles].tolist():
        pairs[order[first : first + count].long()] = e
    got_experts = pairs.view(T, top)
    ranked = torch.sort(z, -1, descending=True).values
    clear = (ranked[:, top - 1] - ranked[:, top]) > 1e-3 if top < experts else torch.ones(T, dtype=torch.bool)
    assert clear.sum() >= T // 2
    assert torch.equal(got_experts[clear].sort(-1).values, chosen[clear].sort(-1).values)
    got_w = route.pair_weight.cpu()[: T * top].view(T, top)
    assert (got_w.sum(-1) - 1).abs().max() <= 1e-5
    for i in torch.nonzero(clear).flatten().tolist():
        by_expert = dict(zip(chosen[i].tolist(), weights[i].tolist()))
        assert all(abs(by_expert[e] - float(a)) <= 2e-5 for e, a in zip(got_experts[i].tolist(), got_w[i]))
    y = part.forward(hd, Step())
    ref = plain.expert_ff(h.double(), wd, "x.", f, False).float()
    tol = (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))
    assert (y.float().cpu() - ref)[clear].abs().max() <= tol
    alone = part.forward(hd[17:18].contiguous(), Step())
    if dtype == "float32":
        assert torch.equal(alone[0], y[17]), "a token's result depends on its company"
    else:
        assert (alone[0].float() - y[17].float()).abs().max() <= tol


def test_router_bias_decides_and_equal_logits_take_the_lower_number():
    from atomserve_amd.kernels import ops

    h = torch.ones(3, 8, device=DEV)
    router = torch.zeros(6, 8, device=DEV)
    bias = torch.tensor([0.0, 2.0, -1.0, 0.0, 2.0, 1.0], device=DEV)
    route = ops.moe_route_scores(h, router, 3, "softmax_of_chosen", bias)
    experts = torch.zeros(9, dtype=torch.int64)
    for e, first, count in route.tiles.cpu()[: int(route.counts.cpu())].tolist():
        experts[route.order.cpu()[first : first + count].long()] = e
    assert experts.view(3, 3).tolist() == [[1, 4, 5]] * 3
    s = torch.softmax(torch.tensor([2.0, 2.0, 1.0]), 0)
    assert torch.allclose(route.pair_weight.cpu().view(3, 3), s.expand(3, 3), atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_reader_of_another_layers_latent_writes_nothing(dtype):
    """Two layers over one latent: the pool has pages for one cache only, and the second layer's logits move when the
    first layer's latent projection changes."""
    raw = copy.deepcopy(CASES["latents"])
    raw["layers"] = raw["layers"][:2]
    weights = random_weights(raw, seed=3)
    model = build_model(raw, weights, dtype)
    requests = model.cache_requests()
    assert len([k for k in requests if not isinstance(k, tuple) and k >= 0]) == 1, "one paged cache for both layers"
    ids = rc.random_ids(raw["vocab"], 40, 1)
    replay = make_replay(raw, weights, dtype, max_tokens=64)
    result = compare(replay, rc.portions("a", ids, sizes=(7, 2, 13)), {"a": ids}, raw, weights, {}, dtype)
    result.check(dtype, "two layers over one latent")
