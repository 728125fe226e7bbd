"""Dozusun on the GPU against the plain implementation (tests/plain_dozusun.py): each mechanism alone, and
whole models of several shapes stepped whole, token by token, in portions down to two tokens, in mixed
batches with pages and state slots used again, and through the engine's scheduler.  Configurations and
weights are made here; where random weights would hide a fault (a window's edge, a far token in a state)
the inputs are made so that it shows."""

import pytest
import torch

from tests import plain_dozusun as plain
from tests import replay_cases as rc
from tests.dozusun_cases import CASES, random_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-5, "bfloat16": 4e-2}


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
    """Engine - plain over many rows, beside what rounding to bfloat16 alone does to the plain model there."""

    def __init__(self):
        self.err, self.noise, self.scale, self.rows = rc.Spread(), rc.Spread(), 1.0, 0

    def add(self, got, exact, rounded=None):
        self.err.add(got - exact)
        if rounded is not None:
            self.noise.add(rounded - exact)
        self.scale = max(self.scale, float(exact.abs().max()))
        self.rows += got.shape[0] if got.dim() > 1 else 1

    def check(self, dtype, what=""):
        """32-bit: rounding of float32 only.  bfloat16: at most what rounding the stored activations moves the plain
        model itself, times 2 in root mean square and 3 at worst (measured: up to 1.8 and 1.3 where few rows are
        compared; the attention kernels also round the softmax's weights before their product with the values,
        which that model does not; a fault of a kernel or a cache moves logits by their own size, tens of times this)."""
        assert self.rows > 0
        if dtype == "float32":
            assert self.err.worst <= TOL[dtype] * self.scale, f"{what}: {self.err.worst:.3e} against |logits| {self.scale:.3e}"
        else:
            assert self.err.rms <= 2.0 * self.noise.rms and self.err.worst <= 3.0 * self.noise.worst, (
                f"{what}: engine - plain rms {self.err.rms:.3e} max {self.err.worst:.3e}; rounding alone "
                f"rms {self.noise.rms:.3e} max {self.noise.worst:.3e}; |logits| {self.scale:.3e}")  # fmt: skip


def reference(raw, weights, ids, refs, key, dtype):
    """(exact logits, logits with bfloat16 activations or None) of a whole sequence, kept in `refs`."""
    if key not in refs:
        refs[key] = (plain.logits(raw, weights, ids), plain.logits(raw, weights, ids, rnd=plain.to_bf16) if dtype == "bfloat16" else None)
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
    free_pages, free_slots = manager.num_free, manager.num_free_slots
    ways = []
    for rid, ids in requests.items():
        ways.append((rid + " whole", rc.whole(rid, ids)))
    ways.append(("a decoded", rc.prefill_then_decode("a", requests["a"], tail=40)))
    ways.append(("b token by token", rc.prefill_then_decode("b", requests["b"], tail=36)))
    ways.append(("a portions", rc.portions("a", requests["a"])))
    ways.append(("e portions of two", rc.portions("e", requests["e"], sizes=(2,))))
    ways.append(("mixed", rc.mixed(requests, seed=7, max_live=3)))
    ways.append(("mixed again", rc.mixed(requests, seed=8, max_live=4, sizes=(2, 3, 16, 17, 5))))
    for name, steps in ways:
        compare(replay, steps, requests, raw, weights, refs, dtype).check(dtype, f"{case} {name}")
        # everything was given back: the next way starts on used pages and slots
        assert manager.num_free == free_pages and manager.num_free_slots == free_slots, name


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_pages_and_windows(dtype):
    """A short prompt and 150 tokens decoded one by one (captured steps): windows, pages of 8 tokens and the
    states all move well past their first borders; a second request decodes beside it from another start."""
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
    and a pool small enough that slots and pages are used again; greedy tokens are the plain model's."""
    from atomserve_amd.config import EngineConfig
    from atomserve_amd.engine.engine import create_engine
    from atomserve_amd.engine.sequence import SamplingParams

    raw = CASES["plain_order"]
    weights = random_weights(raw, seed=33)
    model = build_model(raw, weights, dtype)
    engine = create_engine(model, EngineConfig(block_size=16, num_blocks=24, max_model_len=128, max_num_seqs=2,
                                               max_num_batched_tokens=12))  # fmt: skip
    assert not engine.scheduler.manager.prefix_reuse_possible
    prompts = [rc.random_ids(raw["vocab"], n, 40 + n) for n in (5, 29, 1, 14)]
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True))
    assert engine.scheduler.manager.num_free == 24 and engine.scheduler.manager.num_free_slots == 2
    for prompt, out in zip(prompts, outs):
        assert len(out) == 7
        seq = list(prompt)
        for t in out:
            ref = plain.logits(raw, weights, seq)[-1]
            if dtype == "float32":
                assert t == int(ref.argmax())
            else:
                assert ref[t] >= ref.max() - 8e-2 * max(1.0, float(ref.abs().max()))
            seq.append(t)


# ---- each mechanism alone ---------------------------------------------------------------------------------


def env_for(dtype):
    from atomserve_amd.kernels import ops
    from atomserve_amd.parts.base import BuildEnv

    return BuildEnv(DTYPES[dtype], torch.device(DEV), products=ops.ProductChoices(fixed=True))


def run_mixer(mixer, h, cuts, dtype, block_size=16, slots=3, warm=None):
    """A mixer alone over one request cut into rows of `cuts` tokens; warm: tokens of another request that first
    runs on the same slot and pages and ends, so that what it left must not show."""
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.cache.pools import CachePools
    from atomserve_amd.engine.batch import Row, StepBatch

    asked = mixer.cache_request()
    manager = CacheManager({(0, name): req for name, req in asked.items()}, block_size, 64, slots)
    pools = CachePools(manager, DTYPES[dtype], DEV)
    splits = [s for s in [mixer.row_split()] if s is not None]

    def feed(x, pieces):
        req, at, outs = manager.new_request(), 0, []
        for n in pieces:
            assert manager.reserve(req, at, n)
            batch = StepBatch([Row([0] * n, at, req.tables, [], req.state_slot)], block_size, len(manager.paged_groups), 10,
                              DEV, pools=pools, row_splits=splits)  # fmt: skip
            outs.append(mixer.forward(x[at : at + n].to(DEV).to(DTYPES[dtype]).contiguous(), batch, batch.cache_view(0, True)).float().cpu())
            at += n
            manager.release_behind_window(req, at)
        manager.release(req)
        return torch.cat(outs)

    if warm is not None:
        feed(warm, [warm.shape[0]])
    return feed(h, cuts)


def bf(x):
    return x.bfloat16().float()


def delta_weights(hidden, H, G, D, Dv, taps, gen, rate=0.0):
    def mat(*s, std=0.3):
        return bf(torch.randn(*s, generator=gen) * std)

    return {"q": mat(G * D, hidden), "k": mat(G * D, hidden), "v": mat(H * Dv, hidden), "g": mat(H * Dv, hidden),
            "b": mat(H, hidden), "a": mat(H, hidden), "o": mat(hidden, H * Dv), "q.conv": mat(G * D, taps, std=0.5),
            "k.conv": mat(G * D, taps, std=0.5), "v.conv": mat(H * Dv, taps, std=0.5),
            "A_log": bf(torch.randn(H, generator=gen) * 0.5 + rate), "dt_bias": mat(H), "norm": bf(1 + 0.2 * torch.randn(Dv, generator=gen))}  # fmt: skip


def bind_delta(w, spec, dtype):
    from atomserve_amd.parts.base import build

    part = build("mixer", spec, env_for(dtype))
    t = {"in.weight": torch.cat([w[k] for k in "qkvgba"]), "conv.weight": torch.cat([w[k + ".conv"] for k in "qkv"]),
         "a_log": w["A_log"], "dt_bias": w["dt_bias"], "out_norm.weight": w["norm"], "out.weight": w["o"]}  # fmt: skip
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 4), (3, 3, 136, 72, 2), (2, 1, 64, 8, 1), (8, 2, 128, 128, 3)])
def test_delta_rule_alone(shape, dtype):
    """Heads and widths of several kinds (a key wider than 64 is cut over several lanes, a value head narrower
    than a wave's columns); the request is cut in rows of 1 to 19 tokens on a slot another request used."""
    from atomserve_amd.parts.plan import DeltaRuleSpec, ShortConvSpec

    H, G, D, Dv, taps = shape
    hidden, T = 64, 45
    gen = torch.Generator().manual_seed(sum(shape))
    w = delta_weights(hidden, H, G, D, Dv, taps, gen)
    h = bf(torch.randn(T, hidden, generator=gen))
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "conv": taps}
    ref = plain.gated_delta_mixer(h.double(), {"x." + k: v.double() for k, v in w.items()}, "x.", m, 1e-5).float()
    part = bind_delta(w, DeltaRuleSpec("delta_rule", hidden, H, G, D, Dv, ShortConvSpec(taps), 1e-5), dtype)
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    warm = bf(torch.randn(9, hidden, generator=gen) * 3)
    for cuts in ([T], [1] * T, [19, 1, 2, 2, 1, 17, 3], [2, 43]):
        got = run_mixer(part, h, cuts, dtype, warm=warm)
        assert (got - ref).abs().max() <= tol, f"{shape} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("dim,vdim", [(128, 128), (64, 40), (24, 72), (200, 16)])
def test_delta_scan_however_the_state_is_cut_over_lanes(dim, vdim):
    """The scan cuts a column of the state into 1 to 16 slices by how many rows and heads a step has; every cut that
    a width allows gives the recurrence's result, from a state that another request left and over several rows."""
    from atomserve_amd.kernels import ops

    H, G, gen = 3, 1, torch.Generator().manual_seed(dim + vdim)
    lens, starts, slots = [9, 1, 17], [0, 5, 0], [2, 0, 1]
    T, C = sum(lens), 2 * G * dim + H * vdim
    qkv = torch.randn(T, C, generator=gen)
    qkv[:, : 2 * G * dim] *= dim**-0.5
    beta, decay = torch.rand(T, H, generator=gen), 0.5 + 0.5 * torch.rand(T, H, generator=gen)
    state0 = torch.randn(4, H, dim, vdim, generator=gen)
    want, at = torch.zeros(T, H, vdim, dtype=torch.float64), 0
    final = state0.double().clone()
    for n, start, slot in zip(lens, starts, slots):
        for h in range(H):
            S = final[slot, h].clone() if start > 0 else torch.zeros(dim, vdim, dtype=torch.float64)
            for t in range(at, at + n):
                q, k, v = qkv[t, :dim].double(), qkv[t, dim : 2 * dim].double(), qkv[t, 2 * dim + h * vdim : 2 * dim + (h + 1) * vdim].double()
                S = decay[t, h].double() * S
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
        ops.delta_scan(qkv.to(DEV), G, dim, H, vdim, beta.to(DEV), decay.to(DEV), state, rows, out, slices=slices)
        assert (out.cpu().double() - want).abs().max() <= 2e-5 * float(want.abs().max()), f"{slices} slices"
        assert (state.cpu().double() - final).abs().max() <= 2e-5 * float(final.abs().max()), f"{slices} slices: the state"
        tried += 1
    assert tried >= 4


def test_delta_rule_keeps_a_far_token():
    """With a decay near one and a query that asks for one early token's key, the output hundreds of tokens later
    is that token's value: a state that was lost or restarted on the way shows as a difference of the output's size."""
    from atomserve_amd.parts.plan import DeltaRuleSpec, ShortConvSpec

    H, G, D, Dv, taps, hidden, T = 2, 1, 32, 16, 2, 48, 300
    gen = torch.Generator().manual_seed(5)
    w = delta_weights(hidden, H, G, D, Dv, taps, gen, rate=-9.0)  # exp(A_log) tiny: nearly nothing is forgotten
    w["b"] = w["b"] * 0 + 0.0
    h = bf(torch.randn(T, hidden, generator=gen) * 0.05)
    h[3] = bf(torch.randn(hidden, generator=gen) * 4)  # the early token, far larger than the rest
    h[T - 1] = h[3]
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "conv": taps}
    wd = {"x." + k: v.double() for k, v in w.items()}
    ref = plain.gated_delta_mixer(h.double(), wd, "x.", m, 1e-5).float()
    forgot = plain.gated_delta_mixer(h[100:].double(), wd, "x.", m, 1e-5).float()
    assert (forgot[-1] - ref[-1]).abs().max() > 0.05 * ref[-1].abs().max(), "the far token does not matter in this test"
    part = bind_delta(w, DeltaRuleSpec("delta_rule", hidden, H, G, D, Dv, ShortConvSpec(taps), 1e-5), "float32")
    for cuts in ([T], [150, 149, 1], [7] * 42 + [6], [299, 1]):
        got = run_mixer(part, h, cuts, "float32")
        assert (got - ref).abs().max() <= 5e-5 * max(1.0, float(ref.abs().max())), cuts


def side_weights(hidden, a, r, gen, sharp=False):
    def mat(*s, std=0.3):
        return bf(torch.randn(*s, generator=gen) * std)

    H, G, D, Dv, width, blocks, taps = a["heads"], a["kv_heads"], a["dim"], a["vdim"], r["width"], r["blocks"], r["conv"]
    bw = width // blocks
    w = {"left.q": mat(H * D, hidden), "left.k": mat(G * D, hidden), "left.v": mat(G * Dv, hidden), "left.g": mat(H * Dv, hidden),
         "left.o": mat(hidden, H * Dv), "left.q.norm": bf(1 + 0.2 * torch.randn(D, generator=gen)),
         "left.k.norm": bf(1 + 0.2 * torch.randn(D, generator=gen)),
         "right.y": mat(width, hidden), "right.y.b": mat(width), "right.x": mat(width, hidden), "right.x.b": mat(width),
         "right.conv": mat(width, taps, std=0.5), "right.conv.b": mat(width), "right.ra": mat(blocks, bw, bw), "right.ra.b": mat(blocks, bw),
         "right.ri": mat(blocks, bw, bw), "right.ri.b": mat(blocks, bw), "right.lam": mat(width, std=1.0), "right.o": mat(hidden, width)}  # fmt: skip
    return w


def bind_side(w, spec, dtype):
    from atomserve_amd.parts.base import build

    part = build("mixer", spec, env_for(dtype))
    t = {"in.weight": torch.cat([w[k] for k in ("left.q", "left.k", "left.v", "left.g", "right.y", "right.x")]),
         "out_t.weight": torch.cat([w["left.o"].t(), w["right.o"].t()]), "q_norm.weight": w["left.q.norm"],
         "k_norm.weight": w["left.k.norm"], "y_bias": w["right.y.b"], "x_bias": w["right.x.b"], "conv.weight": w["right.conv"],
         "conv.bias": w["right.conv.b"], "gate_a.weight": w["right.ra"], "gate_a.bias": w["right.ra.b"],
         "gate_i.weight": w["right.ri"], "gate_i.bias": w["right.ri.b"], "lam": w["right.lam"]}  # fmt: skip
    part.bind({k: v.to(DEV).to(DTYPES[dtype]).contiguous() for k, v in t.items()})
    return part


def side_spec(hidden, a, r, left_scale, right_scale, eps=1e-5):
    from atomserve_amd.parts.plan import GatedAttentionSpec, LinearRecurrenceSpec, NormSpec, ShortConvSpec, SideBySideSpec

    return SideBySideSpec("side_by_side", hidden,
                          GatedAttentionSpec(a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["scale"],
                                             NormSpec("rmsnorm", a["dim"], eps), a.get("mask", {}).get("size", 0)),
                          LinearRecurrenceSpec(r["width"], r["blocks"], ShortConvSpec(r["conv"])), left_scale, right_scale)  # fmt: skip


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [
    ({"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.25, "mask": {"size": 7}}, {"width": 40, "blocks": 5, "conv": 4}),
    ({"heads": 3, "kv_heads": 3, "dim": 64, "vdim": 8, "scale": 0.1}, {"width": 72, "blocks": 1, "conv": 1}),
    ({"heads": 6, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 0.2, "mask": {"size": 16}}, {"width": 128, "blocks": 2, "conv": 2}),
])  # fmt: skip
def test_attention_beside_recurrence_alone(sizes, dtype):
    """Keys narrower and wider than values (pages take the wider), a window of 7 and of exactly a page, none at all;
    blocks of 8 to 72 channels; each half also alone (the other's weight zero)."""
    a, r = sizes
    hidden, T = 48, 50
    gen = torch.Generator().manual_seed(a["dim"] + r["width"])
    w = side_weights(hidden, a, r, gen)
    h = bf(torch.randn(T, hidden, generator=gen))
    wd = {"x." + k: v.double() for k, v in w.items()}
    warm = bf(torch.randn(21, hidden, generator=gen) * 2)
    for ls, rs in ((1.25, 0.75), (1.0, 0.0), (0.0, 1.0)):
        m = {"left": a, "right": r, "left_scale": ls, "right_scale": rs}
        ref = plain.side_by_side_mixer(h.double(), wd, "x.", m, 1e-5).float()
        part = bind_side(w, side_spec(hidden, a, r, ls, rs), dtype)
        tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
        for cuts in ([T], [1] * T, [9, 2, 1, 1, 20, 17], [2, 2, 46]):
            got = run_mixer(part, h, cuts, dtype, warm=warm)
            assert (got - ref).abs().max() <= tol, f"{(ls, rs)} {cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("window,block_size", [(12, 16), (16, 16), (17, 8), (1, 16)])
def test_a_window_edge_shows(window, block_size):
    """One token's key matches every later query far better than any other (a sharp softmax), and its value is
    large: while it is inside the window the output is its value, one token later it is gone.  The edge is met
    in a prompt, in a portion that starts just before it, and token by token."""
    a = {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 6.0, "mask": {"size": window}}
    r = {"width": 16, "blocks": 1, "conv": 2}
    hidden, T, mark = 32, 64, 20
    gen = torch.Generator().manual_seed(window)
    w = side_weights(hidden, a, r, gen)
    # queries read the first half of h and keys the second through the same matrix: a token whose second half is
    # the pattern that later tokens carry in their first half is what they all look for
    half = bf(torch.randn(a["dim"], hidden // 2, generator=gen) * 0.5)
    w["left.q"] = torch.cat([torch.cat([half, torch.zeros_like(half)], dim=1)] * a["heads"])
    w["left.k"] = torch.cat([torch.zeros_like(half), half], dim=1)
    h = bf(torch.randn(T, hidden, generator=gen) * 0.3)
    pattern = bf(torch.randn(hidden // 2, generator=gen))
    h[mark + 1 :, : hidden // 2] = pattern
    h[mark, hidden // 2 :] = pattern
    h[mark] = h[mark] * 2  # and its value is large
    m = {"left": a, "right": r, "left_scale": 1.0, "right_scale": 0.0}
    wd = {"x." + k: v.double() for k, v in w.items()}
    ref = plain.side_by_side_mixer(h.double(), wd, "x.", m, 1e-5).float()
    edge = mark + window  # the first position that no longer sees the marked token
    if window > 1:
        wider = dict(m, left=dict(a, mask={"size": window + 1}))
        assert (plain.side_by_side_mixer(h.double(), wd, "x.", wider, 1e-5).float()[edge] - ref[edge]).abs().max() > 0.1 * ref.abs().max()
    part = bind_side(w, side_spec(hidden, a, r, 1.0, 0.0), "float32")
    for cuts in ([T], [edge - 1, 2, T - edge - 1], [mark + 1] + [1] * (T - mark - 1), [edge, 1, T - edge - 1], [3] * 21 + [1]):
        got = run_mixer(part, h, cuts, "float32", block_size=block_size)
        assert (got - ref).abs().max() <= 1e-4 * max(1.0, float(ref.abs().max())), f"window {window} {cuts}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_without_a_window_finds_a_far_key_among_hundreds(dtype):
    """No window: the fourth token's key is what the last tokens look for, 330 tokens and 20 pages later; a page
    lost or a table entry wrong on the way shows at the output's own size.  Met at the end of a long prompt, in a
    portion behind a long cached prefix and token by token."""
    a = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 2.0}
    r = {"width": 16, "blocks": 2, "conv": 2}
    hidden, T, mark = 32, 335, 3
    gen = torch.Generator().manual_seed(77)
    w = side_weights(hidden, a, r, gen)
    half = bf(torch.randn(a["dim"], hidden // 2, generator=gen) * 0.5)
    w["left.q"] = torch.cat([torch.cat([half, torch.zeros_like(half)], dim=1)] * a["heads"])
    w["left.k"] = torch.cat([torch.cat([torch.zeros_like(half), half], dim=1)] * a["kv_heads"])
    h = bf(torch.randn(T, hidden, generator=gen) * 0.3)
    pattern = bf(torch.randn(hidden // 2, generator=gen))
    h[T - 12 :, : hidden // 2] = pattern
    h[mark, hidden // 2 :] = pattern
    h[mark] = h[mark] * 2
    m = {"left": a, "right": r, "left_scale": 1.0, "right_scale": 0.0}
    wd = {"x." + k: v.double() for k, v in w.items()}
    ref = plain.side_by_side_mixer(h.double(), wd, "x.", m, 1e-5).float()
    without = plain.side_by_side_mixer(h[mark + 1 :].double(), wd, "x.", m, 1e-5).float()
    assert (without[-1] - ref[-1]).abs().max() > 0.2 * ref[-1].abs().max(), "the far key does not matter in this test"
    part = bind_side(w, side_spec(hidden, a, r, 1.0, 0.0), dtype)
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    for cuts in ([T], [T - 12, 12], [T - 12] + [1] * 12, [64, 64, 64, 64, 64, 3, 12], [320, 2, 2, 11]):
        got = run_mixer(part, h, cuts, dtype)
        assert (got - ref).abs().max() <= tol, f"{cuts}: {float((got - ref).abs().max()):.3e} of {float(ref.abs().max()):.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,top,ff,T", [(5, 2, 24, 70), (3, 3, 8, 5), (9, 1, 40, 33), (2, 1, 16, 1), (2, 1, 16, 200), (3, 2, 8, 150)])
def test_table_routed_experts_alone(experts, top, ff, T, dtype):
    """From one pair to an expert up to a hundred (several tiles of 64 pairs, the last one partly filled)."""
    from atomserve_amd.engine.batch import Row, StepBatch
    from atomserve_amd.parts.base import build
    from atomserve_amd.parts.plan import TableExpertsSpec

    hidden, vocab = 64, 50
    gen = torch.Generator().manual_seed(experts * 10 + top)
    w = {}
    for e in range(experts):
        w[f"x.e{e}.gate"] = bf(torch.randn(ff, hidden, generator=gen) * 0.3)
        w[f"x.e{e}.up"] = bf(torch.randn(ff, hidden, generator=gen) * 0.3)
        w[f"x.e{e}.down"] = bf(torch.randn(hidden, ff, generator=gen) * 0.3)
    w["x.table"] = torch.rand(vocab, experts, generator=gen).argsort(dim=1)[:, :top].to(torch.int32)
    ids = torch.randint(0, vocab, (T,), generator=gen).tolist()
    h = bf(torch.randn(T, hidden, generator=gen))
    mlp = {"router": {"experts": experts, "top": top}}
    ref = plain.table_routed_experts(h.double(), ids, {k: (v.double() if v.is_floating_point() else v) for k, v in w.items()}, "x.", mlp).float()
    part = build("feed_forward", TableExpertsSpec("table_experts", hidden, ff, experts, top, vocab, "silu"), env_for(dtype))
    dt = DTYPES[dtype]
    part.bind({"gate.weight": torch.stack([w[f"x.e{e}.gate"] for e in range(experts)]).to(DEV).to(dt),
               "up.weight": torch.stack([w[f"x.e{e}.up"] for e in range(experts)]).to(DEV).to(dt),
               "down.weight": torch.stack([w[f"x.e{e}.down"] for e in range(experts)]).to(DEV).to(dt),
               "table": w["x.table"].to(DEV)})  # fmt: skip
    # the tokens as two rows of one step, and each token alone: a token's result does not depend on its company
    cut = max(1, T // 3)
    rows = [Row(ids[:cut], 0, [], [])] + ([Row(ids[cut:], 0, [], [])] if T > cut else [])
    batch = StepBatch(rows, 16, 0, vocab, DEV)
    got = part.forward(h.to(DEV).to(dt), batch).float().cpu()
    tol = (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(ref.abs().max()))
    assert (got - ref).abs().max() <= tol
    for t in range(0, T, 7):
        alone = part.forward(h[t : t + 1].to(DEV).to(dt), StepBatch([Row([ids[t]], 3, [], [])], 16, 0, vocab, DEV)).float().cpu()
        assert torch.equal(alone[0], got[t]), "a token's experts gave another result in other company"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_sum_two_norms(dtype):
    from atomserve_amd.kernels import ops

    gen = torch.Generator().manual_seed(3)
    dt = DTYPES[dtype]
    for n, T in ((96, 5), (520, 3), (4096, 2)):
        x = torch.randn(T, n, generator=gen)
        d1, d2 = bf(torch.randn(T, n, generator=gen)), bf(torch.randn(T, n, generator=gen))
        w1, w2 = bf(1 + 0.1 * torch.randn(n, generator=gen)), bf(1 + 0.1 * torch.randn(n, generator=gen))
        v = x.double() + (d1.double() + d2.double())
        want1 = plain.rms_norm(v, w1.double(), 1e-5).float()
        want2 = plain.rms_norm(v, w2.double(), 1e-5).float()
        xg = x.to(DEV)
        out1, out2 = torch.empty((T, n), dtype=dt, device=DEV), torch.empty((T, n), dtype=dt, device=DEV)
        ops.rmsnorm_multi(xg, w1.to(DEV).to(dt), w2.to(DEV).to(dt), 1e-5, out1, out2, delta1=d1.to(DEV).to(dt), delta2=d2.to(DEV).to(dt))
        tol = 1e-5 if dtype == "float32" else 2e-2
        assert (out1.float().cpu() - want1).abs().max() <= tol * float(want1.abs().max())
        assert (out2.float().cpu() - want2).abs().max() <= tol * float(want2.abs().max())
        assert (xg.cpu() - v.float()).abs().max() <= 1e-6 * float(v.abs().max()), "the stream did not receive the sum in 32 bits"
        rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
        picked = torch.empty((2, n), dtype=dt, device=DEV)
        ops.rmsnorm_multi(xg, w1.to(DEV).to(dt), None, 1e-5, picked, rows=rows, update_x=False)
        assert (picked.float().cpu() - want1[[T - 1, 0]]).abs().max() <= tol * float(want1.abs().max())


def test_short_convolution_and_its_history():
    """Taps of 1 to 5 over rows of every length from a history that another request left: the first tokens of a
    sequence see zeros, a row of one token sees the last taps - 1 inputs of the rows before."""
    from atomserve_amd.kernels import ops

    gen = torch.Generator().manual_seed(9)
    C, T = 70, 23
    for taps in (1, 2, 3, 5):
        w = bf(torch.randn(C, taps, generator=gen))
        bias, in_bias = bf(torch.randn(C, generator=gen)), bf(torch.randn(C, generator=gen))
        x = bf(torch.randn(T, C + 5, generator=gen))
        want = plain.short_conv(x[:, 3 : 3 + C].double() + in_bias.double(), w.double(), bias.double()).float()
        history = torch.randn(4, max(taps - 1, 0), C).to(DEV) * 100  # what an earlier request left in the slots
        for cuts in ([T], [1] * T, [2, 1, 1, 7, 12], [taps, T - taps] if taps < T else [T]):
            got, at = [], 0
            for n in cuts:
                rows = (None if n == 1 else torch.zeros(n, dtype=torch.int32, device=DEV),) + tuple(
                    torch.tensor([v], dtype=torch.int32, device=DEV) for v in (0, n, at, 2))
                out = torch.empty((n, C), dtype=torch.float32, device=DEV)
                ops.short_conv(x[at : at + n].to(DEV).contiguous(), 3, w.to(DEV), history, rows, out, in_bias=in_bias.to(DEV), bias=bias.to(DEV))
                got.append(out.cpu())
                at += n
            assert (torch.cat(got) - want).abs().max() <= 2e-5 * float(want.abs().max()), (taps, cuts)


def test_models_of_these_shapes_say_they_replay():
    """Every part is made of launches on the step's device arrays alone, so decode steps are captured."""
    raw = CASES["looped"]
    assert build_model(raw, random_weights(raw, seed=1), "bfloat16").capturable


def test_the_command_line_generates_from_a_folder(tmp_path, capsys):
    """`atomserve FOLDER --prompt-ids ...` on a Dozusun folder written here: the architecture is found by its name
    in config.json, the weights by their names, and the greedy tokens are the plain model's."""
    import json

    from safetensors.torch import save_file

    from atomserve_amd.engine import cli

    raw = CASES["all_looped"]
    weights = random_weights(raw, seed=17)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    save_file({k: (v if v.dtype == torch.int32 else v.bfloat16()).contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    prompt = rc.random_ids(raw["vocab"], 21, 3)
    code = cli.main([str(tmp_path), "--dtype", "fp32", "--prompt-ids", " ".join(map(str, prompt)), "--max-tokens", "5", "--temperature", "0",
                     "--ignore-eos", "--kv-mem-gb", "0.05", "--max-num-seqs", "2", "--max-batched-tokens", "16"])
    assert code == 0
    lines = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert lines[-1]["output_ids"] == plain.greedy(raw, weights, prompt, 5)
