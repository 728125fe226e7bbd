"""Koravik on the GPU against the plain implementation (tests/plain_koravik.py): each mechanism alone, and
whole models of several shapes stepped whole, token by token, in portions down to two tokens, in mixed
batches with pages used again, and through the engine's scheduler.  Configurations and weights are made
here; where random weights would hide a fault (a window's edge, a kept token, a far key) the inputs are made
so that it shows: one key that every query matches, so the output is its value exactly while it is seen."""

import copy
import json
import os

import pytest
import torch

from tests import plain_koravik as plain
from tests import replay_cases as rc
from tests.koravik_cases import CASES, random_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


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

    def check(self, dtype, what=""):
        """32-bit: rounding of float32 only, at every row.  bfloat16: the rows' errors against what rounding the stored
        activations moves the plain model itself at the same rows, as distributions: the median within 1.5 times that
        model's, the ninth decile within twice its ninth decile.  Rounding moves a router's scores, and where two of
        them lie within that of each other a token takes another expert in one model than in the other (in the plain
        model with rounded activations as well): such rows stand out in both and say nothing about the kernels, which
        the 32-bit runs hold to 3e-5 at every row."""
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_whole_decoded_in_portions_and_mixed(case, dtype):
    """One model, four ways of cutting the same requests: all must give the plain model's logits at every place."""
    raw = CASES[case]
    weights = random_weights(raw, seed=len(case))
    vocab = raw["vocab"]
    requests = {"a": rc.random_ids(vocab, 71, 1), "b": rc.random_ids(vocab, 37, 2), "c": rc.random_ids(vocab, 2, 3),
                "d": rc.random_ids(vocab, 1, 4), "e": rc.random_ids(vocab, 50, 5)}  # fmt: skip
    refs = {}
    replay = make_replay(raw, weights, dtype, max_tokens=4 * 128)
    manager = replay.manager
    free_pages = manager.num_free
    ways = []
    for rid, ids in requests.items():
        ways.append((rid + " whole", rc.whole(rid, ids)))
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
        total.err += result.err
        total.noise += result.noise
        total.scale = max(total.scale, result.scale)
        assert manager.num_free == free_pages, name  # everything was given back: the next way starts on used pages
    total.check(dtype, case)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_whose_mixers_name_no_mask_or_no_rotation(dtype):
    """Without a mask a position sees every earlier key (nothing is given back), without a rotation nothing turns."""
    raw = copy.deepcopy(CASES["wide_groups"])
    raw["layers"][0]["mixer"].pop("mask")
    raw["layers"][1]["mixer"].pop("rot")
    weights = random_weights(raw, seed=12)
    requests = {"a": rc.random_ids(raw["vocab"], 90, 6), "b": rc.random_ids(raw["vocab"], 33, 7)}
    replay = make_replay(raw, weights, dtype, max_tokens=2 * 128, max_live=2)
    refs, total = {}, Against()
    for steps in (rc.whole("a", requests["a"]), rc.portions("a", requests["a"]), rc.mixed(requests, seed=5, max_live=2),
                  rc.prefill_then_decode("b", requests["b"], tail=20)):  # fmt: skip
        result = compare(replay, steps, requests, raw, weights, refs, dtype)
        total.err += result.err
        total.noise += result.noise
        total.scale = max(total.scale, result.scale)
    total.check(dtype, "no mask, no rotation")
    assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [4, 8, 64])
def test_pages_of_other_sizes(block_size, dtype):
    """Windows and kept tokens against pages of 4, 8 and 64 tokens: portions and a mixed batch."""
    raw = CASES["looped"]
    weights = random_weights(raw, seed=9)
    requests = {"a": rc.random_ids(raw["vocab"], 90, 6), "b": rc.random_ids(raw["vocab"], 33, 7), "c": rc.random_ids(raw["vocab"], 70, 8)}
    replay = make_replay(raw, weights, dtype, max_tokens=3 * 128, block_size=block_size, max_live=3)
    refs, total = {}, Against()
    for steps in (rc.portions("a", requests["a"], sizes=(5, 2, 30, 3, 9)), rc.mixed(requests, seed=3, max_live=3),
                  rc.prefill_then_decode("c", requests["c"], tail=45)):  # fmt: skip
        result = compare(replay, steps, requests, raw, weights, refs, dtype)
        total.err += result.err
        total.noise += result.noise
        total.scale = max(total.scale, result.scale)
    total.check(dtype, f"pages of {block_size}")
    assert replay.manager.num_free == replay.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_pages_and_windows(dtype):
    """A short prompt and 150 tokens decoded one by one (captured steps): windows and pages of 8 tokens move well
    past their first borders while the kept tokens stay; a second request decodes beside it from another start."""
    raw = CASES["looped"]
    weights = random_weights(raw, seed=21)
    a, b = rc.random_ids(raw["vocab"], 160, 11), rc.random_ids(raw["vocab"], 90, 12)
    refs = {}
    replay = make_replay(raw, weights, dtype, max_tokens=320, block_size=8)
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
    """The engine's own entry point: prompts of unequal lengths under a small token budget (so prompts are cut)
    and a pool small enough that pages are used again; greedy tokens are the plain model's."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    raw = CASES["all_looped"]
    weights = random_weights(raw, seed=33)
    model = build_model(raw, weights, dtype)
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=24, max_model_len=128, max_num_seqs=2,
                                               max_num_batched_tokens=12))  # fmt: skip
    assert not engine.scheduler.manager.prefix_reuse_possible
    prompts = [rc.random_ids(raw["vocab"], n, 40 + n) for n in (5, 29, 1, 14)]
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True))
    assert engine.scheduler.manager.num_free == 24
    # 32-bit: the plain model's best token.  bfloat16: rounding may send a token to another expert than the plain
    # model's, so the yardstick is the same model stepped whole through the replay tool: its best token, or one as good
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
    """bin/trace_run's own main on a model folder written here: config.json names the architecture."""
    import io

    from safetensors.torch import save_file

    from atomserve_amd.engine import replay

    raw = CASES["wide_groups"]
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
    import numpy as np

    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1))
    assert (got0 - ref[[3, 20]]).abs().max() <= 3e-5 * float(ref.abs().max())
    assert (got1 - ref[[29]]).abs().max() <= 3e-5 * float(ref.abs().max())


def test_the_command_line_generates_from_a_folder_and_from_random_weights(tmp_path, capsys):
    """`atomserve FOLDER --prompt-ids ...` on a Koravik folder written here: the architecture is found by its name
    in config.json, the weights by their names, and the greedy tokens are the plain model's; with
    `--random-weights` the same configuration generates without a checkpoint."""
    from safetensors.torch import save_file

    from atomserve_amd.engine import cli

    raw = CASES["all_looped"]
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


# ---- each mechanism alone ---------------------------------------------------------------------------------


def env_for(dtype):
    from atomserve_amd.kernels import ops
    from atomserve_amd.parts.base import BuildEnv

    return BuildEnv(DTYPES[dtype], torch.device(DEV), products=ops.ProductChoices(fixed=True))


def bf(x):
    return x.bfloat16().float()


def paged(k, v, block_size, gen, dtype, junk=0.0):
    """Keys and values [L, G, D] of one sequence in pages handed out in a random order among others that hold
    `junk`: (k_pages, v_pages, block table [1, pages])."""
    L, G, D = k.shape
    n = -(-L // block_size)
    pool = 2 * n + 3
    order = torch.randperm(pool, generator=gen)[:n]
    kp = torch.full((pool, G, block_size, D), junk)
    vp = torch.full((pool, G, D, block_size), junk)
    for j in range(L):
        kp[order[j // block_size], :, j % block_size] = k[j]
        vp[order[j // block_size], :, :, j % block_size] = v[j]
    t = DTYPES[dtype]
    return kp.to(DEV).to(t), vp.to(DEV).to(t), order.to(torch.int32).view(1, n).to(DEV)


def attend(q, kp, vp, table, mix, scale, window, keep_first, dtype, tile, singles=(), splits=None):
    """The kernel over one sequence whose queries stand at positions 0..L-1: in tiles of `tile` queries, except the
    positions in `singles`, which go as single tokens."""
    from atomserve_amd.kernels import ops

    L, H, D = q.shape
    t = DTYPES[dtype]
    out = torch.zeros((L, H, D), dtype=t, device=DEV)
    qd = q.to(DEV).to(t).contiguous()
    positions = torch.arange(L, dtype=torch.int32, device=DEV)
    rows = torch.zeros(L, dtype=torch.int32, device=DEV)
    mixd = None if mix is None else mix.float().to(DEV).contiguous()
    runs, at = [], 0
    for s in sorted(singles) + [L]:  # the stretches between single tokens, cut into tiles
        for first in range(at, s, tile):
            runs.append((first, min(tile, s - first), 0, first))
        at = s + 1
    if singles:
        items = torch.tensor(sorted(singles), dtype=torch.int32, device=DEV)
        ops.attn_headmix(qd, kp, vp, items, 1, positions, rows, table, mixd, out, scale, window, keep_first,
                         max_context=L, splits=splits)  # fmt: skip
    if runs and tile > 1:
        ops.attn_headmix(qd, kp, vp, torch.tensor(runs, dtype=torch.int32, device=DEV), tile, None, None, table, mixd,
                         out, scale, window, keep_first, max_context=L, splits=splits)  # fmt: skip
    elif runs:
        items = torch.tensor([r[0] for r in runs], dtype=torch.int32, device=DEV)
        ops.attn_headmix(qd, kp, vp, items, 1, positions, rows, table, mixd, out, scale, window, keep_first,
                         max_context=L, splits=splits)  # fmt: skip
    return out.float().cpu()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 6, 24, 8), (18, 1, 8, 4), (16, 2, 64, 64), (3, 1, 40, 16), (32, 4, 128, 16),
                                   (8, 2, 32, 8), (4, 4, 64, 32), (16, 1, 32, 16), (4, 4, 256, 16), (32, 8, 128, 4), (5, 5, 96, 16),
                                   (6, 2, 64, 16), (3, 1, 64, 8), (12, 1, 32, 16)])
def test_mixed_heads_attention_kernel(shape, dtype):
    """Random queries, keys and values over pages in a random order, a window of 37 with 5 kept tokens, a window of
    one, and none: in tiles, as single tokens, and both in one sequence.  In bfloat16 the shapes with heads of a
    multiple of 32 run on the matrix cores (one to sixteen query heads to a kv head, so sixteen to one queries a
    tile), also with an item's keys cut over three workgroups; pages of 4 tokens and the rest run the general kernel,
    which takes an item of more queries than it keeps at once in turns."""
    from atomserve_amd.kernels import ops

    H, G, D, bs = shape
    L, gen = 150, torch.Generator().manual_seed(sum(shape))
    q, k, v = (bf(torch.randn(L, n, D, generator=gen)) for n in (H, G, G))
    mix = bf(torch.eye(H) + 0.4 * torch.randn(H, H, generator=gen))
    kp, vp, table = paged(k, v, bs, gen, dtype, junk=3.0)
    tile = ops.attn_headmix_rows(H, G, D, DTYPES[dtype])
    assert tile >= 1
    on_matrix_cores = ops.attn_headmix_mfma_takes(DTYPES[dtype], H, G, D, bs, tile)
    assert on_matrix_cores == (dtype == "bfloat16" and D % 32 == 0 and bs >= 8 and H // G in (1, 2, 4, 8, 16))
    tol = 2e-5 if dtype == "float32" else 1.5e-2
    for window, keep in ((37, 5), (1, 0), (0, 0), (20, 33)):
        size = window if window else L + 1
        for talk in (mix, None):
            ref = plain.mixed_softmax_attention(q.double(), k.double(), v.double(), talk, D**-0.5, size, keep).float()
            ways = [("tiles", {}), ("single tokens", {"tile": 1}), ("both", {"singles": (0, 7, 8, 64, 149)})]
            if on_matrix_cores:
                ways += [("tiles in three splits", {"splits": 3}), ("both in two splits", {"singles": (1, 63, 148), "splits": 2})]
            for name, kwargs in ways:
                got = attend(q, kp, vp, table, talk, D**-0.5, window, keep, dtype, kwargs.pop("tile", tile), **kwargs)
                assert (got - ref).abs().max() <= tol * float(ref.abs().max()), (
                    f"{shape} window {window} keep {keep} {name}: {float((got - ref).abs().max()):.3e}")  # fmt: skip


@pytest.mark.parametrize("block_size", [8, 16, 64])
def test_window_edges_kept_tokens_and_a_far_key_show(block_size):
    """One key that every query matches far better than any other: while a query sees it, its output is that key's
    value; one position later it is the others'.  The key stands just inside and just outside the window, among the
    kept tokens and right behind them, at a page's border, and hundreds of tokens back; queries come in tiles that
    start anywhere and as single tokens."""
    H, G, D, L = 4, 2, 16, 700
    gen = torch.Generator().manual_seed(block_size)
    unit = torch.zeros(D)
    unit[3] = 1.0
    window, keep = 48, 5
    for special in (4, 5, block_size - 1, block_size, 333, 2 * block_size + 1):
        k = bf(0.05 * torch.randn(L, G, D, generator=gen))
        v = bf(torch.randn(L, G, D, generator=gen))
        k[special] = 30.0 * unit
        v[special] = 9.0
        q = (30.0 * unit).expand(L, H, D).contiguous()
        ref = plain.mixed_softmax_attention(q.double(), k.double(), v.double(), None, 1.0, window, keep).float()
        seen = torch.tensor([special <= i and (i - special < window or special < keep) for i in range(L)])
        assert bool(((ref[seen] - 9.0).abs() < 1e-3).all()) and bool((ref[~seen].abs() < 5.0).all())
        assert bool(seen[special]) and (special < keep) == bool(seen[-1]) and not (special >= keep and bool(seen[special + window]))
        kp, vp, table = paged(k, v, block_size, gen, "float32", junk=7.0)
        edge = min(L - 1, special + window)
        for tile, singles in ((16, ()), (8, (edge - 1, edge, L - 1)), (1, ()), (4, (special, special + 1))):
            got = attend(q, kp, vp, table, None, 1.0, window, keep, "float32", tile, singles)
            assert (got - ref).abs().max() <= 1e-4, f"key at {special}, pages of {block_size}, tiles of {tile}"


def make_attention(raw_mixer, hidden, dtype, gen):
    """The mixer part with random weights, and the same weights under the plain model's names."""
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import MixedHeadsAttentionSpec, RotarySpec

    m = raw_mixer
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    w = {"x.q": bf(0.3 * torch.randn(H * D, hidden, generator=gen)), "x.k": bf(0.3 * torch.randn(G * D, hidden, generator=gen)),
         "x.o": bf(0.2 * torch.randn(hidden, H * D, generator=gen)), "x.talk": bf(torch.eye(H) + 0.3 * torch.randn(H, H, generator=gen)),
         "g": bf(0.2 * torch.randn(hidden, hidden, generator=gen)), "g.b": bf(0.5 * torch.randn(hidden, generator=gen))}  # fmt: skip
    spec = MixedHeadsAttentionSpec(
        "mixed_heads_attention", hidden, H, G, D, m["scale"],
        RotarySpec("rope_half", m["rot"]["dims"], m["rot"]["base"]) if m["rot"]["dims"] else None,
        window=m["mask"]["size"], keep_first=m["mask"]["keep_first"], out_gate=True)  # fmt: skip
    part = build("mixer", spec, env_for(dtype))
    t = {"in.weight": torch.cat([w["x.q"], w["x.k"], w["g"]]), "o.weight": w["x.o"], "mix": w["x.talk"], "gate_bias": w["g.b"]}
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part, w


def run_attention(part, h, cuts, dtype, block_size=16, warm=None):
    """The mixer alone over one request cut into rows of `cuts` tokens, on pages that another request (`warm`) used
    before: returns (outputs, gates) as the part leaves them for the norm that follows."""
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.cache.pools import CachePools
    from atomserve_amd.engine.batch import Row, StepBatch

    manager = CacheManager({0: part.cache_request()}, block_size, 64, 2)
    pools = CachePools(manager, DTYPES[dtype], DEV)

    def feed(x, pieces):
        req, at, ys, gs = manager.new_request(), 0, [], []
        for n in pieces:
            assert manager.reserve(req, at, n)
            batch = StepBatch([Row([0] * n, at, req.tables, [])], block_size, 1, 10, DEV, pools=pools, row_splits=[part.row_split()])
            d = part.forward(x[at : at + n].to(DEV).to(DTYPES[dtype]).contiguous(), batch, batch.cache_view(0, True))
            ys.append(d.y.float().cpu())
            gs.append(torch.sigmoid(d.gate[:, d.gate_off : d.gate_off + x.shape[1]].float() + d.bias.float()).cpu())
            at += n
            manager.release_behind_window(req, at)
        manager.release(req)
        return torch.cat(ys), torch.cat(gs)

    if warm is not None:
        feed(warm, [warm.shape[0]])
    return feed(h, cuts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mixer", [(6, 2, 16, 8, 9, 3), (2, 1, 12, 6, 1, 2), (5, 5, 24, 24, 33, 16), (18, 1, 8, 0, 20, 0), (8, 4, 32, 16, 1000, 0)])
def test_attention_part_alone(mixer, dtype):
    """Heads, groups, widths (12 is padded to 16), turned coordinates (all, half, none), windows and kept tokens of
    several kinds; the request comes whole, token by token and in rows of 1 to 19 tokens, on pages another request
    left, whose pages behind the window are given back on the way."""
    H, G, D, R, size, keep = mixer
    hidden, T = 64, 60
    gen = torch.Generator().manual_seed(sum(mixer))
    m = {"heads": H, "kv_heads": G, "dim": D, "scale": 0.3, "rot": {"dims": R, "base": 77.0}, "mask": {"size": size, "keep_first": keep}}
    part, w = make_attention(m, hidden, dtype, gen)
    h = bf(torch.randn(T, hidden, generator=gen))
    wd = {k: v.double() for k, v in w.items()}
    ref = plain.attention(h.double(), wd, "x.", m).float()
    ref_gate = plain.gate(h.double(), wd, "g").float()
    tol = (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))
    warm = bf(torch.randn(23, hidden, generator=gen) * 3)
    for cuts in ([T], [1] * T, [19, 1, 2, 2, 1, 17, 3, 15], [2, 58]):
        got, gate = run_attention(part, h, cuts, dtype, warm=warm, block_size=8 if len(cuts) == 2 else 16)
        assert (got - ref).abs().max() <= tol, f"{mixer} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"
        assert (gate - ref_gate).abs().max() <= (1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_are_stored_turned_and_values_as_projected(dtype):
    """What the cache holds after a step: the keys turned by their positions (half of a head here), and as values
    the same projections unturned."""
    from atomserve_amd.kernels import ops

    T, H, G, D, R, bs = 21, 3, 1, 16, 8, 8
    gen = torch.Generator().manual_seed(8)
    proj = bf(torch.randn(T, (H + G) * D + 5, generator=gen))
    positions = torch.arange(100, 100 + T)
    t = DTYPES[dtype]
    inv = (1.0 / 50.0 ** (torch.arange(0, R, 2, dtype=torch.float64) / R)).to(DEV)
    table = torch.empty((T, R // 2, 2), dtype=torch.float32, device=DEV)
    ops.rope_table(positions.to(torch.int32).to(DEV), inv, table)
    slots = torch.randperm(6 * bs, generator=gen)[:T].to(torch.int32)
    kp = torch.zeros((6, G, bs, D), dtype=t, device=DEV)
    vp = torch.zeros((6, G, D, bs), dtype=t, device=DEV)
    q = torch.empty((T, H, D), dtype=t, device=DEV)
    ops.head_norm_store(proj.to(DEV).to(t), 0, H * D, H * D, H, G, D, D, None, None, 0.0, slots.to(DEV), q, kp, vp, cos_sin=table)
    want_q = plain.turn_half(proj[:, : H * D].view(T, H, D).double(), positions, R, 50.0).float()
    want_k = plain.turn_half(proj[:, H * D : (H + G) * D].view(T, G, D).double(), positions, R, 50.0).float()
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert (q.float().cpu() - want_q).abs().max() <= tol * float(want_q.abs().max())
    for i in range(T):
        page, off = int(slots[i]) // bs, int(slots[i]) % bs
        assert (kp[page, :, off].float().cpu() - want_k[i]).abs().max() <= tol * float(want_k.abs().max())
        assert torch.equal(vp[page, :, :, off].float().cpu(), proj[i, H * D : (H + G) * D].view(G, D))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(5, 2, 40, 24), (7, 1, 24, 0), (3, 3, 16, 16), (70, 9, 8, 4), (2, 2, 264, 8)])
def test_routed_experts_alone(sizes, dtype):
    """The router's choice and weights against the plain ones, the experts' sum, the shared expert and the gate's
    logits; a token alone gives bit for bit what it gives in company."""
    from atomserve_amd.kernels import ops
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import RoutedExpertsSpec

    experts, top, ff, shared = sizes
    hidden, T = 72, 41
    gen = torch.Generator().manual_seed(sum(sizes))
    w = {"x.router": bf(0.5 * torch.randn(experts, hidden, generator=gen)), "g": bf(0.2 * torch.randn(hidden, hidden, generator=gen)),
         "g.b": bf(0.5 * torch.randn(hidden, generator=gen))}  # fmt: skip
    for e in range(experts):
        w[f"x.e{e}.up"], w[f"x.e{e}.down"] = bf(0.2 * torch.randn(ff, hidden, generator=gen)), bf(0.2 * torch.randn(hidden, ff, generator=gen))
    f = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        w["x.shared.up"], w["x.shared.down"] = bf(0.2 * torch.randn(shared, hidden, generator=gen)), bf(0.2 * torch.randn(hidden, shared, generator=gen))
        f["shared"] = {"ff": shared}
    part = build("feed_forward", RoutedExpertsSpec("routed_experts", hidden, ff, experts, top, "relu2", shared_size=shared, out_gate=True),
                 env_for(dtype))  # fmt: skip
    t = {"router.weight": w["x.router"], "up.weight": torch.stack([w[f"x.e{e}.up"] for e in range(experts)]),
         "down.weight": torch.stack([w[f"x.e{e}.down"] for e in range(experts)]), "gate_bias": w["g.b"],
         "side.weight": torch.cat([w["x.shared.up"], w["g"]]) if shared else w["g"]}  # fmt: skip
    if shared:
        t["shared_down.weight"] = w["x.shared.down"]
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    h = bf(torch.randn(T, hidden, generator=gen))
    wd = {k: v.double() for k, v in w.items()}
    hd = h.to(DEV).to(DTYPES[dtype]).contiguous()

    class Step:
        shared = {}

    route = ops.moe_route_sigmoid(hd, part.router_weight, top)
    torch.cuda.synchronize()
    chosen, weights = plain.route(h.double(), wd["x.router"], top)
    scores = torch.sigmoid(h.double() @ wd["x.router"].T)
    pairs = torch.zeros(T * top, dtype=torch.int64)
    order, tiles, n_tiles = route.order.cpu(), route.tiles.cpu(), int(route.counts.cpu())
    for e, first, count in tiles[:n_tiles].tolist():
        pairs[order[first : first + count].long()] = e
    got_experts = pairs.view(T, top)
    margin = torch.sort(scores, -1, descending=True).values
    clear = (margin[:, top - 1] - margin[:, top]) > 1e-3 if top < experts else torch.ones(T, dtype=torch.bool)
    assert clear.sum() >= T // 2
    assert torch.equal(got_experts[clear].sort(-1).values, chosen[clear].sort(-1).values)
    got_w = route.pair_weight.cpu()[: T * top].view(T, top)
    for i in torch.nonzero(clear).flatten().tolist():
        by_expert = dict(zip(chosen[i].tolist(), weights[i].tolist()))
        assert all(abs(by_expert[e] - float(a)) <= 1e-5 for e, a in zip(got_experts[i].tolist(), got_w[i]))
    d = part.forward(hd, Step())
    ref = plain.experts(h.double(), wd, "x.", f).float()
    tol = (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))
    assert (d.y.float().cpu() - ref)[clear].abs().max() <= tol
    logits = d.gate[:, d.gate_off : d.gate_off + hidden].float().cpu()
    assert (logits - (h.double() @ wd["g"].T).float()).abs().max() <= (1e-5 if dtype == "float32" else 3e-2)
    alone = part.forward(hd[17:18].contiguous(), Step())
    if dtype == "float32":  # every 32-bit product is one chain of multiply-adds per output, whatever the batch
        assert torch.equal(alone.y[0], d.y[17]), "a token's result depends on its company"
    else:  # the dense products of one row and of 41 run through different kernels
        assert (alone.y[0].float() - d.y[17].float()).abs().max() <= tol


def test_router_takes_the_lower_number_of_equal_scores():
    from atomserve_amd.kernels import ops

    h = torch.ones(3, 8, device=DEV)
    router = torch.zeros(6, 8, device=DEV)
    router[4] = 0.5
    router[1] = 0.5
    route = ops.moe_route_sigmoid(h, router, 3)
    experts = torch.zeros(9, dtype=torch.int64)
    for e, first, count in route.tiles.cpu()[: int(route.counts.cpu())].tolist():
        experts[route.order.cpu()[first : first + count].long()] = e
    assert experts.view(3, 3).tolist() == [[1, 4, 0]] * 3
    s = torch.sigmoid(torch.tensor([4.0, 4.0, 0.0]))
    assert torch.allclose(route.pair_weight.cpu().view(3, 3), (s / s.sum()).expand(3, 3), atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", [48, 344, 2056])
def test_gated_sum_norm_and_join(width, dtype):
    """x += m sigmoid(g + b) y in 32 bits, the norm of the sum, rows picked out, the stream left alone where asked,
    and the sum beside another stream as a product's input."""
    from atomserve_amd.kernels import ops

    T, gen = 13, torch.Generator().manual_seed(width)
    t = DTYPES[dtype]
    x = torch.randn(T, width, generator=gen) * 3
    y, gate = bf(torch.randn(T, width, generator=gen)), bf(torch.randn(T, width + 24, generator=gen))
    bias, gain = bf(torch.randn(width, generator=gen)), bf(1 + 0.1 * torch.randn(width, generator=gen))
    other = torch.randn(T, width, generator=gen)
    want_x = x.double() + 0.6 * torch.sigmoid(gate[:, 24:].double() + bias.double()) * y.double()
    want_h = plain.rms_norm(want_x, gain.double(), 1e-5)
    tol = 2e-6 if dtype == "float32" else 1e-2
    dev = lambda a, kind=t: a.to(DEV).to(kind).contiguous()  # noqa: E731
    xs = dev(x, torch.float32)
    out = torch.empty((T, width), dtype=t, device=DEV)
    ops.gated_add_norm(xs, dev(y), dev(gate), 24, dev(bias), 0.6, dev(gain), 1e-5, out)
    assert (xs.cpu().double() - want_x).abs().max() <= 2e-6 * float(want_x.abs().max())
    assert (out.float().cpu().double() - want_h).abs().max() <= tol * float(want_h.abs().max())
    rows = torch.tensor([11, 2, 2, 0], dtype=torch.int32, device=DEV)
    xs = dev(x, torch.float32)
    picked = torch.empty((4, width), dtype=t, device=DEV)
    ops.gated_add_norm(xs, dev(y), dev(gate), 24, dev(bias), 0.6, dev(gain), 1e-5, picked, rows=rows, update_x=False)
    assert torch.equal(xs.cpu(), x) and (picked.float().cpu().double() - want_h[[11, 2, 2, 0]]).abs().max() <= tol * float(want_h.abs().max())
    xs = dev(x, torch.float32)
    join = torch.empty((T, 2 * width), dtype=t, device=DEV)
    ops.gated_add_norm(xs, dev(y), dev(gate), 24, dev(bias), 0.6, None, 0.0, None, other=dev(other, torch.float32), join=join)
    assert (join[:, :width].float().cpu().double() - want_x).abs().max() <= tol * float(want_x.abs().max())
    assert (join[:, width:].float().cpu() - other).abs().max() <= tol * float(other.abs().max())
    plain_norm = torch.empty((T, width), dtype=torch.float32, device=DEV)  # a norm whose result is a stream: 32 bits out
    ops.gated_add_norm(dev(x, torch.float32), None, None, 0, None, 1.0, dev(gain), 1e-5, plain_norm, update_x=False)
    assert (plain_norm.cpu().double() - plain.rms_norm(x.double(), gain.double(), 1e-5)).abs().max() <= 3e-6 * float(x.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_stream_after_every_layer(dtype):
    """The residual stream after every run of a layer (a looped layer counts each time), the pending gated output
    added, against the plain model's: a fault shows at the first layer it touches."""
    raw = CASES["looped"]
    weights = random_weights(raw, seed=4)
    ids = rc.random_ids(raw["vocab"], 45, 3)
    want = []
    plain.forward(ids, raw, {k: v.double() for k, v in weights.items()}, layers_out=want)
    replay = make_replay(raw, weights, dtype, max_tokens=64)
    seen = []
    for block in replay.model.blocks:
        inner = block.forward

        def watched(x, delta, step, cache, next_norm=None, inner=inner):
            d = inner(x, delta, step, cache, next_norm=next_norm)
            g = torch.sigmoid(d.gate[:, d.gate_off : d.gate_off + x.shape[1]].float() + d.bias.float())
            seen.append((x + d.mult * g * d.y.float()).cpu())
            return d

        block.forward = watched
    replay.step([{"id": "a", "tokens": ids, "want": [44]}], ["a"])
    assert len(seen) == len(want) == 7
    rounded = []
    if dtype == "bfloat16":
        plain.forward(ids, raw, {k: v.double() for k, v in weights.items()}, round_to=plain.bf16_round, layers_out=rounded)
    for i, (got, ref) in enumerate(zip(seen, want)):
        rows = (got.double() - ref).abs().max(-1).values
        if dtype == "float32":
            assert float(rows.max()) <= 2e-5 * float(ref.abs().max()), f"run {i}: {float(rows.max()):.3e} of {float(ref.abs().max()):.3e}"
            continue
        # bfloat16: against what rounding the stored activations moves the plain model's own stream after this run
        # (a token whose two best experts score alike may take the other one, and every later run carries that on)
        noise = (rounded[i] - ref).abs().max(-1).values
        assert float(rows.median()) <= 2.0 * float(noise.median()) and float(rows.max()) <= 3.0 * float(noise.max()), (
            f"run {i}: rows' median {float(rows.median()):.3e} and worst {float(rows.max()):.3e}; the plain model's "
            f"{float(noise.median()):.3e} and {float(noise.max()):.3e}")  # fmt: skip
