"""Koravik written plainly: one function per mechanism, whole sequences at once, no cache, sharing
nothing with the package.  `cfg` is the configuration as config.json spells it (a dict), `w` the
checkpoint's tensors by their names; everything is computed in the dtype of `w`'s tensors (float64
in the tests), optionally rounding to bfloat16 at the places where an engine that serves in
bfloat16 stores such numbers (`round_to`), which is the yardstick of the bfloat16 tests.

  stream      x0 = n(E[token]);  per layer  x += m g1 * A(n1 x),  x += m g2 * F(n2 x)
              g = sigmoid(R h + b) with h the sublayer's input;  n(x) = x / sqrt(mean x^2 + eps) * gain
  loop        before layer `start` of each of `times` passes: x <- W_in [x ; x0]
  attention   q = W_q h, k = W_k h, v = k (unturned); first `dims` coordinates of q, k turned by
              p * base^(-2i/dims) in pairs (i, i + dims/2);  s_g = scale q_g . k_kv(g);  s'_h = sum_g T[h, g] s_g;
              j visible from i: j <= i and (i - j < size or j < keep_first);  softmax;  W_o on the heads
  experts     z = W_r h, s = sigmoid z, the `top` largest chosen, weights s / (sum of chosen + 1e-20),
              each expert W_down relu(W_up h)^2; a shared expert of the same form is added
  logits      logit_scale * E n(x)
"""

import math

import torch


def _id(t):
    return t


def bf16_round(t):
    return t.to(torch.bfloat16).to(t.dtype)


def rms_norm(x, gain, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def turn_half(x, positions, dims, base):
    """x [T, heads, D]: the pairs (i, i + dims/2) of the first `dims` coordinates turn by p * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    angle = positions.to(torch.float64)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def visible(T, size, keep_first):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def mixed_softmax_attention(q, k, v, talk, scale, size, keep_first):
    """q [T, H, D], k, v [T, G, D] (positions 0..T-1) -> [T, H, D]: every head's scores are sums of all heads'
    scores weighed by a row of `talk` [H, H] (None: its own only), then masked and softmaxed."""
    T, H, _ = q.shape
    G = k.shape[1]
    kh = k.repeat_interleave(H // G, dim=1)  # head h reads kv head h // (H / G)
    vh = v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kh) * scale
    if talk is not None:
        s = torch.einsum("hg,gij->hij", talk.to(s.dtype), s)
    s = s.masked_fill(~visible(T, size, keep_first)[None], -math.inf)
    return torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), vh)


def attention(h, w, p, m, round_to=_id):
    """h [T, width]; m: the mixer's configuration; p: the tensors' prefix ('l3.mix.')."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = round_to(h @ w[p + "q"].T).view(T, H, D)
    k = round_to(h @ w[p + "k"].T).view(T, G, D)
    v = k  # the keys as projected are the values
    pos = torch.arange(T)
    rot, mask = m.get("rot") or {}, m.get("mask") or {}  # neither: nothing turns, every earlier key is seen
    if rot.get("dims"):
        q = round_to(turn_half(q, pos, rot["dims"], rot["base"]))
        k = round_to(turn_half(k, pos, rot["dims"], rot["base"]))
    o = mixed_softmax_attention(q, k, v, w[p + "talk"], m["scale"], mask.get("size") or T + 1, mask.get("keep_first", 0))
    return round_to(round_to(o).reshape(T, H * D) @ w[p + "o"].T)


def expert(h, up, down, round_to=_id):
    a = round_to(h @ up.T)
    return round_to(round_to(torch.relu(a) ** 2) @ down.T)


def route(h, router, top):
    """Chosen experts [T, top] and their weights."""
    s = torch.sigmoid(h @ router.T)
    chosen = torch.topk(s, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def experts(h, w, p, f, round_to=_id, routes=None):
    """routes: a list that receives (scores of all experts, chosen) per call, for tests that look at margins."""
    T = h.shape[0]
    chosen, weights = route(h, w[p + "router"], f["router"]["top"])
    if routes is not None:
        routes.append((torch.sigmoid(h @ w[p + "router"].T), chosen))
    out = torch.zeros_like(h)
    for t in range(T):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            out[t] += a * expert(h[t : t + 1], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"], round_to)[0]
    if f.get("shared"):
        out = out + expert(h, w[p + "shared.up"], w[p + "shared.down"], round_to)
    return round_to(out)


def gate(h, w, name, round_to=_id):
    return torch.sigmoid(round_to(h @ w[name].T) + w[name + ".b"])


def layer(x, i, cfg, w, round_to=_id):
    c, p, eps, m = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"], cfg["residual_mult"]
    h = round_to(rms_norm(x, w[p + "norm1"], eps))
    x = x + m * gate(h, w, p + "rg1", round_to) * attention(h, w, p + "mix.", c["mixer"], round_to)
    if c["mlp"] is not None:
        h = round_to(rms_norm(x, w[p + "norm2"], eps))
        x = x + m * gate(h, w, p + "rg2", round_to) * experts(h, w, p + "mlp.", c["mlp"], round_to)
    return x


def run_order(cfg):
    """(layer, whether the stream re-enters through the loop's matrix before it) in the order of running."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def logits(cfg, w, tokens, rounded=False):
    """As the other plain models are called: float64 weights from `w`, logits as float32."""
    wd = {k: v.double() for k, v in w.items()}
    return forward(tokens, cfg, wd, round_to=bf16_round if rounded else _id).float()


def forward(tokens, cfg, w, round_to=_id, layers_out=None):
    """Logits [T, vocab] of a whole sequence; layers_out: a list that receives the stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x0 = rms_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    x = x0
    for i, reenter in run_order(cfg):
        if reenter:
            x = round_to(torch.cat([x, x0], dim=-1)) @ w["loop.in"].T
        x = layer(x, i, cfg, w, round_to)
        if layers_out is not None:
            layers_out.append(x)
    h = round_to(rms_norm(x, w["final.norm"], eps))
    return (h @ w["embed"].T) * cfg["logit_scale"]
