"""Small Koravik configurations for the tests, and random weights under the checkpoint's names.

The configurations differ from one another in every size and option: head counts and groups (one kv head for
all, one each, more query heads to a kv head than the kernel takes in one walk), head widths (also ones that
are padded), turned coordinates (all, half, none), windows (one token, less than a page, more than a page, longer
than any request) with 0 to more kept tokens than the window is long (on and off a page's border), experts (all
used, one used, with and without a shared expert), layers without a feed-forward, and a stretch that is absent,
runs once, twice or three times, from the first layer or up to the last."""

import torch


def _attn(heads, kv_heads, dim, scale, rot_dims, base, size, keep_first):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
            "rot": {"dims": rot_dims, "base": base}, "mask": {"size": size, "keep_first": keep_first}}  # fmt: skip


def _moe(ff, experts, top, shared=0):
    raw = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        raw["shared"] = {"ff": shared}
    return raw


CASES = {
    # a stretch of two layers runs three times; half of a head turns; more kept tokens than the window is long
    "looped": {
        "architecture": "Koravik", "vocab": 300, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 0.6, "logit_scale": 2.0,
        "layers": [
            {"type": "attention", "mixer": _attn(6, 2, 16, 0.3, 8, 10000.0, 9, 3), "mlp": _moe(40, 5, 2, shared=24)},
            {"type": "attention", "mixer": _attn(3, 3, 24, 0.25, 24, 500.0, 21, 0), "mlp": _moe(24, 7, 1)},
            {"type": "attention", "mixer": _attn(8, 1, 8, 0.4, 4, 100.0, 5, 7), "mlp": None},
        ],
        "loop": {"start": 1, "stop": 3, "times": 3},
    },  # fmt: skip
    # no loop at all; a window longer than any request; a window of one token; every expert used; padded heads; nothing turns
    "plain_order": {
        "architecture": "Koravik", "vocab": 128, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 1.0, "logit_scale": 0.25,
        "layers": [
            {"type": "attention", "mixer": _attn(4, 4, 32, 0.2, 32, 300000.0, 1000, 0), "mlp": _moe(16, 3, 3, shared=16)},
            {"type": "attention", "mixer": _attn(2, 1, 12, 0.5, 6, 50.0, 1, 2), "mlp": _moe(8, 2, 1, shared=8)},
            {"type": "attention", "mixer": _attn(2, 2, 8, 0.35, 0, 10.0, 6, 1), "mlp": None},
        ],
    },  # fmt: skip
    # the whole model is one stretch that runs twice (the first run enters through the loop's matrix); kept tokens
    # that fill a page exactly; a window longer than two pages
    "all_looped": {
        "architecture": "Koravik", "vocab": 200, "width": 80, "norm": {"eps": 1e-5}, "residual_mult": 0.8, "logit_scale": 1.0,
        "layers": [
            {"type": "attention", "mixer": _attn(5, 5, 16, 0.25, 16, 1000.0, 17, 16), "mlp": None},
            {"type": "attention", "mixer": _attn(4, 2, 20, 0.3, 10, 20000.0, 33, 1), "mlp": _moe(24, 9, 4, shared=32)},
        ],
        "loop": {"start": 0, "stop": 2, "times": 2},
    },  # fmt: skip
    # a stretch of one layer that runs once, up to the last layer; 18 query heads on one kv head; 16 heads in groups of 8
    "wide_groups": {
        "architecture": "Koravik", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "residual_mult": 0.5, "logit_scale": 1.5,
        "layers": [
            {"type": "attention", "mixer": _attn(16, 2, 8, 0.35, 8, 300.0, 12, 4), "mlp": _moe(8, 4, 2)},
            {"type": "attention", "mixer": _attn(18, 1, 8, 0.3, 2, 7.0, 40, 0), "mlp": _moe(12, 2, 2, shared=4)},
        ],
        "loop": {"start": 1, "stop": 2, "times": 1},
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

    w = {"embed": mat(vocab, h, s=1.0), "embed.norm": gain(h), "final.norm": gain(h)}
    if raw.get("loop"):
        w["loop.in"] = mat(h, 2 * h, s=1.0 / (2 * h) ** 0.5 * 1.5)
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = gain(h)
        w[p + "rg1"], w[p + "rg1.b"] = mat(h, h), mat(h, s=0.5)
        x = p + "mix."
        w[x + "q"], w[x + "k"] = mat(m["heads"] * m["dim"], h, s=0.3), mat(m["kv_heads"] * m["dim"], h, s=0.3)
        w[x + "talk"] = (torch.eye(m["heads"]) + 0.3 * torch.randn(m["heads"], m["heads"], generator=g)).bfloat16().float()
        w[x + "o"] = mat(h, m["heads"] * m["dim"])
        mlp = layer["mlp"]
        if mlp is None:
            continue
        w[p + "norm2"] = gain(h)
        w[p + "rg2"], w[p + "rg2.b"] = mat(h, h), mat(h, s=0.5)
        x = p + "mlp."
        ff, experts = mlp["expert"]["ff"], mlp["router"]["experts"]
        for e in range(experts):
            w[f"{x}e{e}.up"], w[f"{x}e{e}.down"] = mat(ff, h), mat(h, ff)
        w[x + "router"] = mat(experts, h, s=0.3)
        if mlp.get("shared"):
            w[x + "shared.up"], w[x + "shared.down"] = mat(mlp["shared"]["ff"], h), mat(h, mlp["shared"]["ff"])
    return w
