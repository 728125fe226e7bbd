"""Small Dozusun configurations for the tests, and random weights under the checkpoint's names.

The configurations differ from one another in every size and option: head counts and groups, key and value
widths (equal, keys wider, values wider), windows (none, one token, a few, more than a page), taps of the
convolutions (1 to 4), blocks of the recurrence's gates (1 to 5), dense and routed feed-forwards and none,
experts used per token (1 to 3), the order of the layers, and a stretch that runs one, two or three times."""

import torch


def _side(heads, kv_heads, dim, vdim, scale, window, width, blocks, conv, left_scale, right_scale):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window}
    return {"left": left, "left_scale": left_scale, "right": {"width": width, "blocks": blocks, "conv": conv},
            "right_scale": right_scale}  # fmt: skip


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


CASES = {
    # a stretch of two layers runs three times; a layer without a feed-forward; values wider than keys
    "looped": {
        "architecture": "Dozusun", "vocab": 300, "width": 96, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "parallel", "mixer": _side(6, 2, 16, 24, 0.3, 9, 48, 3, 2, 1.1, 0.8), "mlp": _moe(40, 5, 2)},
            {"type": "delta", "mixer": _delta(6, 3, 24, 16, 3), "mlp": {"kind": "dense", "ff": 72}},
            {"type": "delta", "mixer": _delta(2, 2, 40, 8, 1), "mlp": None},
        ],
        "loop": {"start": 1, "stop": 3, "times": 3},
    },  # fmt: skip
    # no loop; no window; a window of one token; every expert used by every token; one kv head
    "plain_order": {
        "architecture": "Dozusun", "vocab": 128, "width": 64, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "delta", "mixer": _delta(4, 1, 8, 32, 4), "mlp": _moe(16, 3, 3)},
            {"type": "parallel", "mixer": _side(4, 4, 32, 16, 0.2, 0, 64, 1, 4, 0.7, 1.3), "mlp": None},
            {"type": "parallel", "mixer": _side(2, 1, 8, 8, 0.5, 1, 32, 4, 1, 1.0, 1.0), "mlp": {"kind": "dense", "ff": 24}},
        ],
    },  # fmt: skip
    # the whole model is one stretch that runs twice; a window longer than a page; keys of 72 in a delta layer
    "all_looped": {
        "architecture": "Dozusun", "vocab": 200, "width": 80, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "parallel", "mixer": _side(5, 5, 16, 16, 0.25, 21, 80, 5, 3, 1.0, 0.5), "mlp": {"kind": "dense", "ff": 56}},
            {"type": "delta", "mixer": _delta(3, 1, 72, 24, 2), "mlp": _moe(24, 7, 1)},
        ],
        "loop": {"start": 0, "stop": 2, "times": 2},
    },  # fmt: skip
    # delta layers only (no pages at all), widths that are no multiples of 4 or 8, an odd number of heads
    "delta_only": {
        "architecture": "Dozusun", "vocab": 90, "width": 44, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "delta", "mixer": _delta(3, 3, 6, 10, 2), "mlp": _moe(12, 4, 2)},
            {"type": "delta", "mixer": _delta(5, 1, 18, 6, 3), "mlp": {"kind": "dense", "ff": 20}},
        ],
        "loop": {"start": 1, "stop": 2, "times": 2},
    },  # fmt: skip
    # side-by-side layers only, more query heads to a kv head than a matrix tile holds rows for (17), one block a channel
    "side_only": {
        "architecture": "Dozusun", "vocab": 64, "width": 48, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "parallel", "mixer": _side(17, 1, 8, 4, 0.35, 5, 24, 24, 2, 0.9, 1.1), "mlp": _moe(8, 2, 1)},
            {"type": "parallel", "mixer": _side(2, 2, 12, 20, 0.3, 33, 40, 2, 3, 1.0, 1.0), "mlp": None},
        ],
    },  # fmt: skip
}


def random_weights(raw: dict, seed: int, std: float = 0.15) -> dict:
    """Tensors under the checkpoint's names, float32 holding bfloat16 values (exact in both precisions)."""
    g = torch.Generator().manual_seed(seed)
    h, vocab = raw["width"], raw["vocab"]

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16().float()

    def gain(n):
        return (1.0 + torch.randn(n, generator=g) * 0.1).bfloat16().float()

    w = {"embed": mat(vocab, h, s=1.0), "final.norm": gain(h), "head": mat(vocab, h)}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = gain(h)
        if layer["type"] == "delta":
            x = p + "mix."
            for name, rows in (("q", m["kv_heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["heads"] * m["vdim"])):
                w[x + name] = mat(rows, h)
                w[x + name + ".conv"] = mat(rows, m["conv"], s=0.5)
            w[x + "g"], w[x + "o"] = mat(m["heads"] * m["vdim"], h), mat(h, m["heads"] * m["vdim"])
            w[x + "b"], w[x + "a"] = mat(m["heads"], h), mat(m["heads"], h)
            w[x + "A_log"], w[x + "dt_bias"] = mat(m["heads"], s=0.5), mat(m["heads"], s=0.5)
            w[x + "norm"] = gain(m["vdim"])
        else:
            a, r, x = m["left"], m["right"], p + "mix.left."
            w[x + "q"], w[x + "k"] = mat(a["heads"] * a["dim"], h), mat(a["kv_heads"] * a["dim"], h)
            w[x + "v"], w[x + "g"] = mat(a["kv_heads"] * a["vdim"], h), mat(a["heads"] * a["vdim"], h)
            w[x + "o"] = mat(h, a["heads"] * a["vdim"])
            w[x + "q.norm"], w[x + "k.norm"] = gain(a["dim"]), gain(a["dim"])
            x, bw = p + "mix.right.", r["width"] // r["blocks"]
            w[x + "y"], w[x + "y.b"] = mat(r["width"], h), mat(r["width"])
            w[x + "x"], w[x + "x.b"] = mat(r["width"], h), mat(r["width"])
            w[x + "conv"], w[x + "conv.b"] = mat(r["width"], r["conv"], s=0.5), mat(r["width"])
            w[x + "ra"], w[x + "ra.b"] = mat(r["blocks"], bw, bw), mat(r["blocks"], bw)
            w[x + "ri"], w[x + "ri.b"] = mat(r["blocks"], bw, bw), mat(r["blocks"], bw)
            w[x + "lam"], w[x + "o"] = mat(r["width"], s=1.0), mat(h, r["width"])
        mlp = layer["mlp"]
        if mlp is None:
            continue
        w[p + "norm2"] = gain(h)
        x = p + "mlp."
        if mlp["kind"] == "dense":
            w[x + "gate"], w[x + "up"], w[x + "down"] = mat(mlp["ff"], h), mat(mlp["ff"], h), mat(h, mlp["ff"])
        else:
            ff, experts, top = mlp["expert"]["ff"], mlp["router"]["experts"], mlp["router"]["top"]
            for e in range(experts):
                w[f"{x}e{e}.gate"], w[f"{x}e{e}.up"], w[f"{x}e{e}.down"] = mat(ff, h), mat(ff, h), mat(h, ff)
            w[x + "table"] = torch.rand(vocab, experts, generator=g).argsort(dim=1)[:, :top].to(torch.int32)
    return w
