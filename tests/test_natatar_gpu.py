"""Natatar on the GPU against the plain implementation (tests/plain_natatar.py): each mechanism alone, and whole
models of several shapes stepped whole, token by token, in portions down to two tokens, in mixed batches with pages
and state slots used again, and through the engine's scheduler.  Configurations and weights are made here; where
random weights would hide a fault (a far key among hundreds, a page's border, a slot that another request left
full, a gate that never saturates) the inputs are made so that it shows."""

import json
import math
import os

import pytest
import torch

from tests import plain_natatar as plain
from tests import replay_cases as rc
from tests.natatar_cases import CASES, random_weights

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
        rounding the stored activations moves the plain model itself at the same rows (a token whose router scores lie
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
    raw = CASES["two_streams"]
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
    raw = CASES["wide_heads"] if dtype == "bfloat16" else CASES["one_stream"]
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

    raw = CASES["two_streams"]
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
    """The replay tool's own main on a model folder written here: config.json names the architecture, and the ranks of
    the delta rule's two-step projections, which this config.json does not name, are read from the tensors' shapes."""
    import io

    import numpy as np
    from safetensors.torch import save_file

    from atomserve_amd.engine import replay

    raw = json.loads(json.dumps(CASES["plain_sums"]))
    weights = random_weights(raw, seed=17)
    for layer in raw["layers"]:
        layer["mixer"].pop("decay_rank", None)
        layer["mixer"].pop("gate_rank", None)
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
    ref = plain.logits(CASES["plain_sums"], weights, ids)
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    assert (got0 - ref[[3, 20]]).abs().max() <= 3e-5 * float(ref.abs().max())
    assert (got1 - ref[[29]]).abs().max() <= 3e-5 * float(ref.abs().max())


def test_the_command_line_generates_from_a_folder_and_from_random_weights(tmp_path, capsys):
    from safetensors.torch import save_file

    from atomserve_amd.engine import cli

    raw = CASES["one_stream"]
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
@pytest.mark.parametrize("case", ["two_streams", "plain_sums"])
def test_the_stream_after_every_layer(case, dtype):
    """The sum of the streams after every layer against the plain model's: a fault shows at the first layer it touches."""
    raw = CASES[case]
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

        def watched(x, delta, step, *a, inner=inner, **k):
            d = inner(x, delta, step, *a, **k)
            xs = step.shared["streams"].double()
            if d is None:  # the last layer leaves the sum as the stream
                seen.append(x.double().cpu())
            else:  # the layer's last write is still pending: done here as the equations say
                mix = d.mix.double() if d.mix is not None else torch.eye(xs.shape[1], dtype=torch.float64, device=xs.device)
                new = torch.einsum("sr,tsn->trn", mix, xs) + d.mult * d.out.double().view(1, -1, 1) * d.y.double().unsqueeze(1)
                seen.append(new.sum(1).cpu())
            return d

        block.forward = watched
    replay.step([{"id": "a", "tokens": ids, "want": [44]}], ["a"])
    assert len(seen) == len(want) == len(raw["layers"])
    for i, (got, ref) in enumerate(zip(seen, want)):
        rows = (got - ref).abs().max(-1).values
        if dtype == "float32":
            assert float(rows.max()) <= 2e-5 * float(ref.abs().max()), f"layer {i}: {float(rows.max()):.3e} of {float(ref.abs().max()):.3e}"
            continue
        noise = (rounded[i] - ref).abs().max(-1).values
        assert float(rows.median()) <= 2.0 * float(noise.median()) and float(rows.quantile(0.9)) <= 2.0 * float(noise.quantile(0.9)), (
            f"layer {i}: rows' median {float(rows.median()):.3e} and ninth decile {float(rows.quantile(0.9)):.3e}; the plain "
            f"model's {float(noise.median()):.3e} and {float(noise.quantile(0.9)):.3e}")  # fmt: skip


# ---- each mechanism alone -------------------------------------------------------------------------------------


def env_for(dtype):
    from atomserve_amd.kernels import ops
    from atomserve_amd.parts.base import BuildEnv

    return BuildEnv(DTYPES[dtype], torch.device(DEV), products=ops.ProductChoices(fixed=True))


def bf(x):
    return x.bfloat16().float()


def run_mixers(mixers, inputs, cuts, dtype, block_size=16, slots=3, warm=None):
    """Mixers alone (each with caches of its own, one after the other in every step, sharing the step's results) over
    one request cut into rows of `cuts` tokens; warm: how many tokens another request first runs on the same slot and
    pages before it ends, so that what it left must not show.  Returns each mixer's outputs [T, hidden]."""
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.cache.pools import CachePools
    from atomserve_amd.engine.batch import Row, StepBatch

    asked = {(i, name): req for i, mixer in enumerate(mixers) for name, req in mixer.cache_request().items()}
    manager = CacheManager(asked, block_size, 64, slots)
    pools = CachePools(manager, DTYPES[dtype], DEV)
    splits = sorted({s for s in [m.row_split() for m in mixers] if s is not None})

    def feed(xs, pieces):
        req, at, outs = manager.new_request(), 0, [[] for _ in mixers]
        for n in pieces:
            assert manager.reserve(req, at, n)
            batch = StepBatch([Row([0] * n, at, req.tables, [], req.state_slot)], block_size, len(manager.paged_groups), 10,
                              DEV, pools=pools, row_splits=splits)  # fmt: skip
            for i, (mixer, x) in enumerate(zip(mixers, xs)):
                y = mixer.forward(x[at : at + n].to(DEV).to(DTYPES[dtype]).contiguous(), batch, batch.cache_view(i, True))
                outs[i].append(y.float().cpu())
            at += n
        manager.release(req)
        return [torch.cat(o) for o in outs]

    if warm:
        gen = torch.Generator().manual_seed(warm)
        feed([bf(torch.randn(warm, x.shape[1], generator=gen) * 3) for x in inputs], [warm])
    return feed(inputs, cuts)


def attention_weights(hidden, m, gen, biased, gated, std=0.3):
    def mat(*s, sd=std):
        return bf(torch.randn(*s, generator=gen) * sd)

    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    w = {"q": mat(H * D, hidden), "k": mat(G * D, hidden), "v": mat(G * E, hidden), "o": mat(hidden, H * E)}
    if biased:
        w.update({"q.b": mat(H * D), "k.b": mat(G * D), "v.b": mat(G * E), "q.norm": bf(2 + 0.3 * torch.randn(H * D, generator=gen)),
                  "k.norm": bf(2 + 0.3 * torch.randn(G * D, generator=gen)), "vmix": bf(torch.tensor(0.35))})  # fmt: skip
    if gated:
        w["g"] = mat(H * E, hidden)
    return w


def bind_attention(w, hidden, m, dtype, biased, gated, value_mix="none", scale=1.0):
    """One softmax core as a mixer of its own."""
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import JoinedMixerSpec, NeighbourRotarySpec, SoftmaxCoreSpec

    rot = m.get("rot")
    position = None
    if rot:
        sc = rot.get("scaling")
        position = NeighbourRotarySpec("rope_neighbours", rot["dims"], rot["base"], *((sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else ()))
    core = SoftmaxCoreSpec("softmax_core", m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], bias=biased,
                           whole_norm_eps=1e-5 if biased else 0.0, position=position, value_mix=value_mix, out_gate=gated)  # fmt: skip
    part = build("mixer", JoinedMixerSpec("joined", hidden, (core,), (scale,)), env_for(dtype))
    t = {"in.weight": torch.cat([w[k] for k in (("q", "k", "v", "g") if gated else ("q", "k", "v"))]), "out_t.weight": w["o"].t()}
    if biased:
        t.update({"c0.q_bias": w["q.b"], "c0.k_bias": w["k.b"], "c0.v_bias": w["v.b"], "c0.q_norm": w["q.norm"], "c0.k_norm": w["k.norm"]})
    if value_mix == "later":
        t["c0.value_mix"] = w["vmix"]
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part


ATTENTIONS = [
    # heads, kv heads, keys, values, biased and normed over the whole projection, rotation (turned, base, scaling), gated
    (4, 2, 16, 24, True, None, False),
    (3, 3, 8, 8, True, None, False),
    (8, 2, 32, 32, True, None, False),
    (2, 1, 128, 64, True, None, False),
    (6, 3, 96, 96, False, (96, 300000.0, (6.0, 32, 8.0, 1.5)), True),
    (2, 1, 32, 16, False, (16, 10000.0, (4.0, 64, 16.0, 2.0)), True),
    (3, 3, 10, 14, False, (10, 500.0, None), True),
    (4, 1, 64, 64, False, (2, 50.0, None), False),
    (5, 5, 24, 8, False, None, True),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ATTENTIONS)
def test_softmax_core_alone(shape, dtype):
    """Biases, the norm over the whole projection, the rotation of neighbours (whole heads, parts of heads, stretched
    or not) and the output gate, each in several sizes, in rows of 1 to 19 tokens on pages another request left."""
    H, G, D, E, biased, rot, gated = shape
    hidden, T = 64, 45
    gen = torch.Generator().manual_seed(H * 100 + D)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "scale": D**-0.5}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
        if rot[2]:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot[2]))
    w = attention_weights(hidden, m, gen, biased, gated)
    h = bf(torch.randn(T, hidden, generator=gen))
    wd = {"x." + k: v.double() for k, v in w.items()}
    if biased:
        ref = plain.attention_mixer(h.double(), wd, "x.", m, 1e-5, False, {}).float()
    else:
        if not gated:
            wd["x.g"] = torch.zeros(H * E, hidden, dtype=torch.float64)  # sigmoid(0): half of the heads
        ref = plain.gated_rotary_attention(h.double(), wd, "x.", m, torch.arange(T), False).float()
    part = bind_attention(w, hidden, m, dtype, biased, gated, scale=1.0 if gated or biased else 0.5)
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    for cuts in ([T], [1] * T, [19, 1, 2, 2, 1, 17, 3], [2, 43]):
        (got,) = run_mixers([part], [h], cuts, dtype, warm=9)
        assert (got - ref).abs().max() <= tol, f"{shape} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_values_mixed_with_the_first_layers(dtype):
    """Three attentions of different head counts whose values have one shape: the first keeps its values, the others
    mix theirs with them before they are cached (each with a weight of its own), also for tokens that come one by one
    or in portions: what is mixed in is the first layer's value of the same token."""
    hidden, T = 48, 40
    gen = torch.Generator().manual_seed(3)
    shapes = [{"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "v_mix": True},
              {"heads": 4, "kv_heads": 4, "dim": 8, "vdim": 12, "scale": 0.35, "v_mix": True},  # other heads, the same projection size
              {"heads": 6, "kv_heads": 2, "dim": 32, "vdim": 24, "scale": 0.18, "v_mix": True}]  # fmt: skip
    ws = [attention_weights(hidden, m, gen, True, False) for m in shapes]
    ws[2]["vmix"] = bf(torch.tensor(0.8))
    hs = [bf(torch.randn(T, hidden, generator=gen)) for _ in shapes]
    shared, refs = {}, []
    for m, w, h in zip(shapes, ws, hs):
        refs.append(plain.attention_mixer(h.double(), {"x." + k: v.double() for k, v in w.items()}, "x.", m, 1e-5, False, shared).float())
    alone = plain.attention_mixer(hs[2].double(), {"x." + k: v.double() for k, v in ws[2].items()}, "x.", dict(shapes[2], v_mix=False), 1e-5, False, {}).float()
    assert (alone - refs[2]).abs().max() > 0.1 * refs[2].abs().max(), "the mixing does not matter in this test"
    parts = [bind_attention(w, hidden, m, dtype, True, False, value_mix=mix) for m, w, mix in zip(shapes, ws, ("first", "later", "later"))]
    for cuts in ([T], [1] * T, [17, 2, 1, 20], [2] * 20):
        got = run_mixers(parts, hs, cuts, dtype, warm=5)
        for i, (g, ref) in enumerate(zip(got, refs)):
            tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
            assert (g - ref).abs().max() <= tol, f"layer {i} {cuts}: {float((g - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("block_size", [8, 16, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_and_keys_at_page_borders(block_size, dtype):
    """One token's key matches the last queries far better than any other (a sharp softmax), and its value is large:
    330 tokens and many pages later the output is its value, and a page lost or a table entry wrong on the way shows at
    the output's own size.  The token stands at the first place of a sequence, at the last place of a page, at the
    first of the next, and its readers come at the end of a long prompt, in a portion behind a long cached prefix and
    token by token."""
    m = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 2.0}
    hidden, T = 32, 335
    for mark in (0, 3, block_size - 1, block_size, 5 * block_size - 1):
        gen = torch.Generator().manual_seed(77 + mark)
        w = attention_weights(hidden, m, gen, True, False)
        for name in ("q.b", "k.b", "v.b"):
            w[name] = torch.zeros_like(w[name])
        half = bf(torch.randn(m["dim"], hidden // 2, generator=gen) * 0.5)
        w["q"] = torch.cat([torch.cat([half, torch.zeros_like(half)], dim=1)] * m["heads"])
        w["k"] = torch.cat([torch.cat([torch.zeros_like(half), half], dim=1)] * m["kv_heads"])
        w["q.norm"], w["k.norm"] = torch.full_like(w["q.norm"], 2.0), torch.full_like(w["k.norm"], 2.0)
        h = bf(torch.randn(T, hidden, generator=gen) * 0.3)
        pattern = bf(torch.randn(hidden // 2, generator=gen))
        h[T - 12 :, : hidden // 2] = pattern
        h[mark, hidden // 2 :] = pattern
        h[mark] = h[mark] * 2
        wd = {"x." + k: v.double() for k, v in w.items()}
        ref = plain.attention_mixer(h.double(), wd, "x.", m, 1e-5, False, {}).float()
        if mark < T - 13:
            hidden_mark = h.clone()
            hidden_mark[mark] = 0
            without = plain.attention_mixer(hidden_mark.double(), wd, "x.", m, 1e-5, False, {}).float()
            assert (without[-1] - ref[-1]).abs().max() > 0.2 * ref[-1].abs().max(), "the far key does not matter in this test"
        part = bind_attention(w, hidden, m, dtype, True, False)
        # bfloat16: a sharp softmax over rounded queries and keys; a lost key changes the output by its own size
        tol = (3e-5 if dtype == "float32" else 1e-1) * max(1.0, float(ref.abs().max()))
        for cuts in ([T], [T - 12, 12], [T - 12] + [1] * 12, [mark + 1, T - 13 - mark, 2, 10], [64, 64, 64, 64, 64, 3, 12]):
            (got,) = run_mixers([part], [h], [c for c in cuts if c > 0], dtype, block_size=block_size, warm=20)
            assert (got - ref).abs().max() <= tol, f"mark {mark} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


def memory_weights(hidden, m, gen):
    def mat(*s, sd=0.3):
        return bf(torch.randn(*s, generator=gen) * sd)

    H, D, E = m["heads"], m["dim"], m["vdim"]
    return {"q": mat(H * D, hidden), "k": mat(H * D, hidden), "v": mat(H * E, hidden), "g": mat(H * E, hidden), "o": mat(hidden, H * E),
            "norm": bf(1 + 0.2 * torch.randn(H * E, generator=gen)), "i": mat(H, hidden), "i.b": mat(H, sd=0.5), "f": mat(H, hidden),
            "f.b": bf(2 + torch.randn(H, generator=gen))}  # fmt: skip


def bind_memory(w, hidden, m, dtype, scale=1.0):
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import JoinedMixerSpec, MatrixMemorySpec

    core = MatrixMemorySpec("matrix_memory", m["heads"], m["dim"], m["vdim"], m["gate_cap"], 1e-5)
    part = build("mixer", JoinedMixerSpec("joined", hidden, (core,), (scale,)), env_for(dtype))
    t = {"in.weight": torch.cat([w[k] for k in ("q", "k", "v", "g", "i", "f")]), "out_t.weight": w["o"].t(), "c0.i_bias": w["i.b"],
         "c0.f_bias": w["f.b"], "c0.out_norm": w["norm"]}  # fmt: skip
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 8, 24, 10.0), (1, 80, 8, 5.0), (2, 64, 64, 18.0), (2, 200, 16, 30.0), (4, 40, 56, 12.0), (5, 6, 6, 2.0)])
def test_matrix_memory_alone(shape, dtype):
    """Heads and widths of several kinds (keys wider than a lane's slice, values narrower than a wave's columns, a cap
    that the gates reach); the request is cut in rows of 1 to 19 tokens on a slot another request used."""
    H, D, E, cap = shape
    hidden, T = 64, 45
    gen = torch.Generator().manual_seed(int(H * 100 + D + cap))
    m = {"heads": H, "dim": D, "vdim": E, "gate_cap": cap}
    w = memory_weights(hidden, m, gen)
    if cap < 5:
        w["i"], w["f"] = w["i"] * 8, w["f"] * 8  # logits well beyond the cap
    h = bf(torch.randn(T, hidden, generator=gen))
    ref = plain.matrix_memory_mixer(h.double(), {"x." + k: v.double() for k, v in w.items()}, "x.", m, 1e-5, False).float()
    part = bind_memory(w, hidden, m, dtype)
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    for cuts in ([T], [1] * T, [19, 1, 2, 2, 1, 17, 3], [2, 43]):
        (got,) = run_mixers([part], [h], cuts, dtype, warm=9)
        assert (got - ref).abs().max() <= tol, f"{shape} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("dim,vdim", [(128, 128), (64, 40), (24, 72), (200, 16), (8, 8)])
def test_memory_scan_however_the_state_is_cut_over_lanes(dim, vdim):
    """Every cut of a column of the state over lanes that a width allows gives the recurrence's result, from states,
    normalisers and maxima that another request left, over several rows of one step; gates from far below zero to
    their cap, so that the maximum moves and the bound e^(-m) of the denominator is met on both sides."""
    from atomserve_amd.kernels import ops

    H, gen = 3, torch.Generator().manual_seed(dim + vdim)
    lens, starts, slots = [9, 1, 17], [0, 5, 0], [2, 0, 1]
    T, C = sum(lens), 2 * H * dim + H * vdim
    qkv = torch.randn(T, C, generator=gen)
    qkv[:, : 2 * H * dim] *= dim**-0.5
    i_log = torch.randn(T, H, generator=gen) * 4
    f_log = -torch.rand(T, H, generator=gen) * 3
    state0, norm0 = torch.randn(4, H, dim, vdim, generator=gen), torch.randn(4, H, dim, generator=gen)
    max0 = torch.randn(4, H, generator=gen) * 2
    want, at = torch.zeros(T, H, vdim, dtype=torch.float64), 0
    S_end, n_end, m_end = state0.double().clone(), norm0.double().clone(), max0.double().clone()
    for n, start, slot in zip(lens, starts, slots):
        rows = slice(at, at + n)
        q = qkv[rows, : H * dim].double().view(n, H, dim)
        k = qkv[rows, H * dim : 2 * H * dim].double().view(n, H, dim)
        v = qkv[rows, 2 * H * dim :].double().view(n, H, vdim)
        S = S_end[slot].clone() if start > 0 else torch.zeros(H, dim, vdim, dtype=torch.float64)
        nn = n_end[slot].clone() if start > 0 else torch.zeros(H, dim, dtype=torch.float64)
        mm = m_end[slot].clone() if start > 0 else torch.zeros(H, dtype=torch.float64)
        for t in range(n):
            fl, il = f_log[at + t].double(), i_log[at + t].double()
            m_new = torch.maximum(fl + mm, il)
            keep, take = torch.exp(fl + mm - m_new), torch.exp(il - m_new)
            S = keep.view(H, 1, 1) * S + take.view(H, 1, 1) * k[t].unsqueeze(2) * v[t].unsqueeze(1)
            nn = keep.view(H, 1) * nn + take.view(H, 1) * k[t]
            mm = m_new
            den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
            want[at + t] = torch.einsum("hde,hd->he", S, q[t]) / den.unsqueeze(1)
        S_end[slot], n_end[slot], m_end[slot] = S, nn, mm
        at += n
    firsts = [sum(lens[:i]) for i in range(len(lens))]
    rows = (None,) + tuple(torch.tensor(v, dtype=torch.int32, device=DEV) for v in (firsts, lens, starts, slots))
    tried = 0
    for slices in (0, 1, 2, 4, 8, 16):
        if slices and -(-dim // slices) > 32:
            continue
        state, norm, mx = state0.clone().to(DEV), norm0.clone().to(DEV), max0.clone().to(DEV)
        out = torch.empty((T, H, vdim), dtype=torch.float32, device=DEV)
        ops.memory_scan(qkv.to(DEV), H, dim, vdim, i_log.to(DEV), f_log.to(DEV), state, norm, mx, rows, out, slices=slices)
        assert (out.cpu().double() - want).abs().max() <= 2e-5 * float(want.abs().max()), f"{slices} slices"
        for name, got, end in (("state", state, S_end), ("normaliser", norm, n_end), ("maximum", mx, m_end)):
            assert (got.cpu().double() - end).abs().max() <= 2e-5 * float(end.abs().max()), f"{slices} slices: the {name}"
        tried += 1
    assert tried >= 3


def test_matrix_memory_keeps_a_far_token():
    """One early token opens its input gate to the cap while all others keep theirs far below, and nothing is
    forgotten: hundreds of tokens later a query that asks for its key reads its value.  A state, normaliser or maximum
    that was lost or restarted on the way shows as a difference of the output's size."""
    H, D, E, hidden, T = 2, 32, 16, 48, 300
    m = {"heads": H, "dim": D, "vdim": E, "gate_cap": 12.0}
    gen = torch.Generator().manual_seed(5)
    w = memory_weights(hidden, m, gen)
    w["i"], w["f"] = w["i"] * 0, w["f"] * 0
    w["i"][:, 0] = 4.0  # the first coordinate of a token's input opens its input gate
    w["i.b"], w["f.b"] = torch.full((H,), -6.0), torch.full((H,), 12.0)
    h = bf(torch.randn(T, hidden, generator=gen) * 0.3)
    h[:, 0] = 0.0
    h[3, 0] = 8.0
    h[T - 1, 1:] = h[3, 1:]
    wd = {"x." + k: v.double() for k, v in w.items()}
    ref = plain.matrix_memory_mixer(h.double(), wd, "x.", m, 1e-5, False).float()
    forgot = plain.matrix_memory_mixer(h[100:].double(), wd, "x.", m, 1e-5, False).float()
    assert (forgot[-1] - ref[-1]).abs().max() > 0.2 * ref[-1].abs().max(), "the far token does not matter in this test"
    part = bind_memory(w, hidden, m, "float32")
    for cuts in ([T], [150, 149, 1], [7] * 42 + [6], [299, 1], [4, 296], [3, 1, 296]):
        (got,) = run_mixers([part], [h], cuts, "float32", warm=11)
        assert (got - ref).abs().max() <= 2e-4 * max(1.0, float(ref.abs().max())), cuts  # weights of e^12 beside e^0 in 32 bits


def channel_delta_weights(hidden, m, gen, rate=0.0):
    def mat(*s, sd=0.3):
        return bf(torch.randn(*s, generator=gen) * sd)

    H, G, D, E, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    return {"q": mat(G * D, hidden), "k": mat(G * D, hidden), "v": mat(H * E, hidden), "b": mat(H, hidden), "o": mat(hidden, H * E),
            "q.conv": mat(G * D, taps, sd=0.5), "k.conv": mat(G * D, taps, sd=0.5), "v.conv": mat(H * E, taps, sd=0.5),
            "A_log": bf(torch.randn(H, generator=gen) * 0.5 + rate), "dt_bias": bf(torch.randn(H * D, generator=gen) - 1.0),
            "a1": mat(m["decay_rank"], hidden), "a2": mat(H * D, m["decay_rank"], sd=0.6), "g1": mat(m["gate_rank"], hidden),
            "g2": mat(H * E, m["gate_rank"], sd=0.6), "norm": bf(1 + 0.2 * torch.randn(E, generator=gen))}  # fmt: skip


def bind_channel_delta(w, hidden, m, dtype):
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import ChannelDeltaRuleSpec, ShortConvSpec

    spec = ChannelDeltaRuleSpec("channel_delta_rule", hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], ShortConvSpec(m["conv"]),
                                m["decay_rank"], m["gate_rank"], 1e-5)  # fmt: skip
    part = build("mixer", spec, env_for(dtype))
    t = {"in.weight": torch.cat([w[k] for k in "qkvb"]), "low.weight": torch.cat([w["a1"], w["g1"]]), "decay_up.weight": w["a2"],
         "gate_up.weight": w["g2"], "conv.weight": torch.cat([w[k + ".conv"] for k in "qkv"]), "a_log": w["A_log"],
         "dt_bias": w["dt_bias"], "out_norm.weight": w["norm"], "out.weight": w["o"]}  # fmt: skip
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 24, 16, 3, 5, 7), (3, 3, 136, 72, 2, 8, 8), (2, 1, 64, 8, 1, 3, 9), (8, 2, 128, 128, 4, 16, 24),
                                   (3, 3, 10, 14, 5, 4, 4)])  # fmt: skip
def test_channel_delta_rule_alone(shape, dtype):
    H, G, D, E, taps, ra, rg = shape
    hidden, T = 64, 45
    gen = torch.Generator().manual_seed(sum(shape))
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "conv": taps, "decay_rank": ra, "gate_rank": rg}
    w = channel_delta_weights(hidden, m, gen)
    h = bf(torch.randn(T, hidden, generator=gen))
    ref = plain.channel_delta_mixer(h.double(), {"x." + k: v.double() for k, v in w.items()}, "x.", m, 1e-5, False).float()
    part = bind_channel_delta(w, hidden, m, dtype)
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    for cuts in ([T], [1] * T, [19, 1, 2, 2, 1, 17, 3], [2, 43]):
        (got,) = run_mixers([part], [h], cuts, dtype, warm=9)
        assert (got - ref).abs().max() <= tol, f"{shape} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("dim,vdim", [(128, 128), (64, 40), (24, 72), (200, 16), (10, 6)])
def test_delta_scan_with_decays_per_channel_however_the_state_is_cut(dim, vdim):
    """Decays that differ from channel to channel (from 0.05 to 1) act on the rows of the state that belong to them;
    every cut of a column over lanes gives the recurrence's result from a state another request left."""
    from atomserve_amd.kernels import ops

    H, G, gen = 4, 2, torch.Generator().manual_seed(dim + vdim)
    lens, starts, slots = [9, 1, 17], [0, 5, 0], [2, 0, 1]
    T, C = sum(lens), 2 * G * dim + H * vdim
    qkv = torch.randn(T, C, generator=gen)
    qkv[:, : 2 * G * dim] *= dim**-0.5
    beta = torch.rand(T, H, generator=gen)
    chan = 0.05 + 0.95 * torch.rand(T, H, dim, generator=gen)
    state0 = torch.randn(4, H, dim, vdim, generator=gen)
    want, at = torch.zeros(T, H, vdim, dtype=torch.float64), 0
    final = state0.double().clone()
    for n, start, slot in zip(lens, starts, slots):
        for h in range(H):
            g = h // (H // G)
            S = final[slot, h].clone() if start > 0 else torch.zeros(dim, vdim, dtype=torch.float64)
            for t in range(at, at + n):
                q, k = qkv[t, g * dim : (g + 1) * dim].double(), qkv[t, (G + g) * dim : (G + g + 1) * dim].double()
                v = qkv[t, 2 * G * dim + h * vdim : 2 * G * dim + (h + 1) * vdim].double()
                S = chan[t, h].double().unsqueeze(1) * S
                S = S + torch.outer(k, beta[t, h].double() * (v - S.T @ k))
                want[t, h] = S.T @ q
            final[slot, h] = S
        at += n
    firsts = [sum(lens[:i]) for i in range(len(lens))]
    rows = (None,) + tuple(torch.tensor(v, dtype=torch.int32, device=DEV) for v in (firsts, lens, starts, slots))
    tried = 0
    for slices in (0, 1, 2, 4, 8, 16):
        if slices and -(-dim // slices) > 64:
            continue
        state = state0.clone().to(DEV)
        out = torch.empty((T, H, vdim), dtype=torch.float32, device=DEV)
        ops.delta_scan_channels(qkv.to(DEV), G, dim, H, vdim, beta.to(DEV), chan.to(DEV), state, rows, out, slices=slices)
        assert (out.cpu().double() - want).abs().max() <= 2e-5 * float(want.abs().max()), f"{slices} slices"
        assert (state.cpu().double() - final).abs().max() <= 2e-5 * float(final.abs().max()), f"{slices} slices: the state"
        tried += 1
    assert tried >= 4


def test_channel_delta_rule_keeps_a_far_token():
    """With decays near one and a query that asks for one early token's key, the output hundreds of tokens later is
    that token's value: a state that was lost or restarted on the way shows as a difference of the output's size."""
    H, G, D, E, taps, hidden, T = 2, 1, 32, 16, 2, 48, 300
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "conv": taps, "decay_rank": 4, "gate_rank": 4}
    gen = torch.Generator().manual_seed(5)
    w = channel_delta_weights(hidden, m, gen, rate=-9.0)  # exp(A_log) tiny: nearly nothing is forgotten
    w["b"] = w["b"] * 0
    h = bf(torch.randn(T, hidden, generator=gen) * 0.05)
    h[3] = bf(torch.randn(hidden, generator=gen) * 4)  # the early token, far larger than the rest
    h[T - 1] = h[3]
    wd = {"x." + k: v.double() for k, v in w.items()}
    ref = plain.channel_delta_mixer(h.double(), wd, "x.", m, 1e-5, False).float()
    forgot = plain.channel_delta_mixer(h[100:].double(), wd, "x.", m, 1e-5, False).float()
    assert (forgot[-1] - ref[-1]).abs().max() > 0.05 * ref[-1].abs().max(), "the far token does not matter in this test"
    part = bind_channel_delta(w, hidden, m, "float32")
    for cuts in ([T], [150, 149, 1], [7] * 42 + [6], [299, 1]):
        (got,) = run_mixers([part], [h], cuts, "float32", warm=11)
        assert (got - ref).abs().max() <= 5e-5 * max(1.0, float(ref.abs().max())), cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(1, 40), (2, 96), (3, 256), (4, 1032), (8, 40), (3, 9000), (2, 4101), (5, 16400), (16, 24)])
def test_streams_are_written_read_and_normed_in_one_pass(sizes, dtype):
    from atomserve_amd.kernels import ops

    S, n = sizes
    T, gen = 5, torch.Generator().manual_seed(S * n)
    x0 = torch.randn(T, n, generator=gen) * 3
    mix, out_c, in_c = torch.eye(S) + 0.3 * torch.randn(S, S, generator=gen), torch.randn(S, generator=gen), torch.rand(S, generator=gen) + 0.2
    gain = 1 + 0.2 * torch.randn(n, generator=gen)
    y = bf(torch.randn(T, n, generator=gen))
    dt = DTYPES[dtype]
    tol = 1e-5 if dtype == "float32" else 1e-2
    xs = torch.empty((T, S, n), dtype=torch.float32, device=DEV)
    h = torch.empty((T, n), dtype=dt, device=DEV)
    # the first read: every stream is what the embedding gave
    ops.streams_step(xs, first=x0.to(DEV), in_c=in_c.to(DEV), gain=gain.to(DEV), eps=1e-5, normed=h)
    ref_xs = x0.double().unsqueeze(0).repeat(S, 1, 1)
    assert torch.equal(xs.cpu(), ref_xs.float().transpose(0, 1))
    want = plain.rms(plain.streams_read(ref_xs, in_c.double()), 1e-5) * gain.double()
    assert (h.float().cpu() - want).abs().max() <= tol * float(want.abs().max())
    # a pending write, the next read and its norm
    ops.streams_step(xs, y=y.to(DEV).to(dt), mix=mix.to(DEV), out_c=out_c.to(DEV), mult=0.45, in_c=in_c.to(DEV), gain=gain.to(DEV), eps=1e-5, normed=h)
    ref_xs = plain.streams_write(ref_xs, mix.double(), out_c.double(), 0.45, y.double())
    assert (xs.cpu().double().transpose(0, 1) - ref_xs).abs().max() <= 1e-5 * float(ref_xs.abs().max())
    want = plain.rms(plain.streams_read(ref_xs, in_c.double()), 1e-5) * gain.double()
    assert (h.float().cpu() - want).abs().max() <= tol * float(want.abs().max())
    # the last write leaves the sum of the streams
    total = torch.empty((T, n), dtype=torch.float32, device=DEV)
    ops.streams_step(xs, y=y.to(DEV).to(dt), mix=None, out_c=out_c.to(DEV), mult=1.0, total=total)
    ref_xs = plain.streams_write(ref_xs, torch.eye(S, dtype=torch.float64), out_c.double(), 1.0, y.double())
    assert (total.cpu().double() - ref_xs.sum(0)).abs().max() <= 1e-5 * float(ref_xs.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_router_scores_groups_and_weights(dtype):
    """The softmax over all experts, the groups of neighbours of which the best are kept, the `top` largest among
    them, weights that are scores times a factor; ties go to the lower number."""
    from atomserve_amd.kernels import ops

    gen = torch.Generator().manual_seed(2)
    for experts, groups, keep, top, K in ((12, 3, 2, 3, 64), (6, 3, 1, 2, 40), (8, 1, 1, 8, 24), (70, 7, 3, 5, 96), (4, 4, 2, 2, 17), (9, 3, 3, 1, 64)):
        T = 33
        h, router = bf(torch.randn(T, K, generator=gen)), bf(torch.randn(experts, K, generator=gen) * 0.5)
        s = torch.softmax(h.double() @ router.double().t(), dim=-1)
        want = plain.grouped_choice(s, top, groups, keep)
        route = ops.moe_route_scores(h.to(DEV).to(DTYPES[dtype]), router.to(DEV).to(DTYPES[dtype]), top, "softmax", None, groups, keep, 2.5)
        # the pairs' experts are not handed back by the route; the order holds every pair once, and the tiles name the experts
        order, tiles, count = route.order.cpu(), route.tiles.cpu(), int(route.counts.cpu())
        got = torch.full((T * top,), -1, dtype=torch.long)
        for e, first, n in tiles[:count].tolist():
            got[order[first : first + n].long()] = e
        got = got.view(T, top)
        # scores within rounding of each other may change places between float64 and float32: rows whose choice differs
        # between the two precisions of the plain router itself are left out
        s32 = torch.softmax(h @ router.t(), dim=-1)
        clear = (plain.grouped_choice(s32.double(), top, groups, keep).sort(-1).values == want.sort(-1).values).all(-1)
        assert clear.sum() >= T - 3
        assert torch.equal(got[clear].sort(-1).values, want[clear].sort(-1).values), (experts, groups, keep, top)
        weights = route.pair_weight.cpu().view(T, top)
        ref_w = 2.5 * torch.gather(s, 1, got.clamp_min(0))
        assert (weights[clear].double() - ref_w[clear]).abs().max() <= 1e-5
    # equal scores: the lower group, and within it the lower expert
    h = torch.zeros(2, 16)
    route = ops.moe_route_scores(h.to(DEV).to(DTYPES[dtype]), torch.zeros(6, 16).to(DEV).to(DTYPES[dtype]), 2, "softmax", None, 3, 2, 1.0)
    tiles, count = route.tiles.cpu(), int(route.counts.cpu())
    assert sorted(e for e, _, n in tiles[:count].tolist() for _ in range(n)) == [0, 0, 1, 1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(6, 2, 40, 24, 3, 2), (4, 4, 24, 8, 1, 1), (9, 3, 16, 16, 3, 1), (12, 3, 264, 96, 3, 2)])
def test_experts_with_groups_alone(sizes, dtype):
    """The feed-forward of experts alone against the plain one; in 32-bit a token alone gives bit for bit what it gives
    in company (every output is one chain of multiply-adds over the whole width, whatever else is in the step)."""
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import GatedRoutedExpertsSpec

    experts, top, hidden, ff, groups, keep = sizes
    gen = torch.Generator().manual_seed(sum(sizes))
    W = {"x.router": bf(torch.randn(experts, hidden, generator=gen) * 0.5)}
    for e in range(experts):
        W[f"x.e{e}.gate"], W[f"x.e{e}.up"] = bf(torch.randn(ff, hidden, generator=gen) * 0.3), bf(torch.randn(ff, hidden, generator=gen) * 0.3)
        W[f"x.e{e}.down"] = bf(torch.randn(hidden, ff, generator=gen) * 0.3)
    raw = {"expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": 1.5, "groups": {"count": groups, "keep": keep}}}
    T = 70
    h = bf(torch.randn(T, hidden, generator=gen))
    ref = plain.experts(h.double(), {k: v.double() for k, v in W.items()}, "x.", raw, False).float()
    spec = GatedRoutedExpertsSpec("gated_routed_experts", hidden, ff, experts, top, "silu", 0.0, score="softmax", router_bias=False,
                                  groups=groups, keep_groups=keep, weight_scale=1.5)  # fmt: skip
    part = build("feed_forward", spec, env_for(dtype))
    t = {"router.weight": W["x.router"]}
    for name in ("gate", "up", "down"):
        t[name + ".weight"] = torch.stack([W[f"x.e{e}.{name}"] for e in range(experts)])
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    hd = h.to(DEV).to(DTYPES[dtype])
    got = part.forward(hd, None).float().cpu()
    rows = (got - ref).abs().max(-1).values
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    assert (rows <= tol).sum() >= T - 2, "a token whose scores lie within rounding of each other may take another expert"
    if dtype == "float32":
        for t_ in (0, 17, 69):
            assert torch.equal(part.forward(hd[t_ : t_ + 1].contiguous(), None).float().cpu()[0], got[t_])


def test_models_of_these_shapes_say_they_replay():
    for case in sorted(CASES):
        assert build_model(CASES[case], random_weights(CASES[case], seed=1), "bfloat16").capturable
