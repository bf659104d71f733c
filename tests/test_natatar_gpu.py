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
