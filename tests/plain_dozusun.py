"""The Dozusun decoder, plainly: one slow function per mechanism, whole sequences, no cache, no
batches, written from the design's equations alone (it shares no code with the package).

A model is a raw configuration (the dict of config.json) and a dict of tensors under the
checkpoint's own names; everything is computed in the dtype of the tensors handed in (the tests
hand in float64).  Token by token where the design is a recurrence, so that nothing here can be
wrong in the way a chunked or batched kernel can.

`rnd` (default: nothing) is applied wherever an engine that computes its matrix products in bfloat16
must store a bfloat16 number: the normed rows, what a product gives and what the next one takes, the
keys, queries and values of the attention.  With `rnd = to_bf16` the model's own logits move by what
rounding alone does, which is the yardstick of the bfloat16 tests; nothing that enters a recurrence
after the projections is rounded.
"""

import math

import torch


def keep(x):
    return x


def to_bf16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def short_conv(x, weight, bias=None):
    """Causal convolution per channel over time: x [T, C], weight [C, taps] whose last column
    multiplies the current token; zeros stand before the first token."""
    T, C = x.shape
    taps = weight.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                out[t] += weight[:, j] * x[src]
    if bias is not None:
        out = out + bias
    return out


def windowed_attention(q, k, v, scale, window):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query head h reads kv head h // (H / G); position i
    sees j with 0 <= i - j < window (window 0: every j <= i).  Returns [T, H, Dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window <= 0 else max(0, i - window + 1)
            s = (k[lo : i + 1, g] @ q[i, h]) * scale
            p = torch.softmax(s, dim=0)
            out[i, h] = p @ v[lo : i + 1, g]
    return out


def gated_attention(h, w, p, m, eps, rnd=keep):
    """The attention half of the side-by-side mixer: per-head RMS norm of q and k, no rotation, a
    sliding window, and sigmoid(W_g h) on the concatenated heads before the output projection."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(h @ w[p + "q"].T).view(T, H, D)
    k = rnd(h @ w[p + "k"].T).view(T, G, D)
    v = rnd(h @ w[p + "v"].T).view(T, G, Dv)
    q = rnd(rms_norm(q, w[p + "q.norm"], eps))
    k = rnd(rms_norm(k, w[p + "k.norm"], eps))
    window = int((m.get("mask") or {}).get("size", 0))
    o = rnd(windowed_attention(q, k, v, m["scale"], window)).reshape(T, H * Dv)
    return o * torch.sigmoid(rnd(h @ w[p + "g"].T))  # what the output projection takes


def gated_linear_recurrence(h, w, p, m, rnd=keep):
    """The recurrent half: y = gelu(W_y h + b), u = conv(W_x h + b); per block of channels two gates
    from square matrices; a = exp(-8 r softplus(lam)); S = a S + sqrt(1 - a^2) i u from S = 0; W_o (S y)."""
    T = h.shape[0]
    width, blocks = m["width"], m["blocks"]
    y = gelu_tanh(rnd(h @ w[p + "y"].T) + w[p + "y.b"])
    u = short_conv(rnd(h @ w[p + "x"].T) + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    bw = width // blocks
    ub = u.view(T, blocks, bw)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, width)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, width)
    log_a = -8.0 * r * softplus(w[p + "lam"])
    a = torch.exp(log_a)
    s = torch.zeros(width, dtype=h.dtype)
    out = torch.zeros(T, width, dtype=h.dtype)
    for t in range(T):
        s = a[t] * s + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = s * y[t]
    return out  # what the output projection takes


def side_by_side_mixer(h, w, p, m, eps, rnd=keep):
    left = rnd(m["left_scale"] * gated_attention(h, w, p + "left.", m["left"], eps, rnd))
    right = rnd(m["right_scale"] * gated_linear_recurrence(h, w, p + "right.", m["right"], rnd))
    return rnd(left @ w[p + "left.o"].T + right @ w[p + "right.o"].T)


def gated_delta_mixer(h, w, p, m, eps, rnd=keep):
    """Gated delta rule per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(rnd(h @ w[p + "q"].T), w[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(rnd(h @ w[p + "k"].T), w[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(rnd(h @ w[p + "v"].T), w[p + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * D**-0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(rnd(h @ w[p + "b"].T))
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(rnd(h @ w[p + "a"].T) + w[p + "dt_bias"]))
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    o = o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w[p + "norm"]
    o = rnd(o.reshape(T, H * Dv) * silu(rnd(h @ w[p + "g"].T)))
    return rnd(o @ w[p + "o"].T)


def dense_feed_forward(h, w, p, rnd=keep):
    return rnd(rnd(silu(rnd(h @ w[p + "gate"].T)) * rnd(h @ w[p + "up"].T)) @ w[p + "down"].T)


def table_routed_experts(h, ids, w, p, mlp, rnd=keep):
    """Every token id names its experts in a table; each chosen expert weighs 1 / top."""
    top = mlp["router"]["top"]
    out = torch.zeros_like(h)
    table = w[p + "table"]
    for t in range(h.shape[0]):
        for j in range(top):
            q = f"{p}e{int(table[int(ids[t]), j])}."
            act = rnd(silu(rnd(h[t] @ w[q + "gate"].T)) * rnd(h[t] @ w[q + "up"].T))
            out[t] += (act @ w[q + "down"].T) / top  # the experts' outputs meet unrounded
    return rnd(out)


def run_order(raw):
    """Indices of the layers in the order they run: a stretch may run several times in a row."""
    n = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(raw, w, ids, streams=None, rnd=keep):
    """Logits [T, vocab] of a whole sequence.  streams: a list that receives the residual stream
    after every layer run."""
    ids = torch.as_tensor(ids)
    eps = raw["norm"]["eps"]
    x = w["embed"][ids]
    for i in run_order(raw):
        layer, p = raw["layers"][i], f"l{i}."
        h1 = rnd(rms_norm(x, w[p + "norm1"], eps))
        if layer["type"] == "delta":
            mixed = gated_delta_mixer(h1, w, p + "mix.", layer["mixer"], eps, rnd)
        elif layer["type"] == "parallel":
            mixed = side_by_side_mixer(h1, w, p + "mix.", layer["mixer"], eps, rnd)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h2 = rnd(rms_norm(x, w[p + "norm2"], eps))
            if mlp["kind"] == "dense":
                mixed = mixed + dense_feed_forward(h2, w, p + "mlp.", rnd)
            else:
                mixed = mixed + table_routed_experts(h2, ids, w, p + "mlp.", mlp, rnd)
        x = x + mixed
        if streams is not None:
            streams.append(x.clone())
    x = rnd(rms_norm(x, w["final.norm"], eps))
    return x @ w["head"].T


def logits(raw, w, ids, rnd=keep):
    return forward(raw, {k: (v.double() if v.is_floating_point() else v) for k, v in w.items()}, ids, rnd=rnd).float()


def greedy(raw, w, prompt, count):
    seq = list(prompt)
    for _ in range(count):
        seq.append(int(logits(raw, w, seq)[-1].argmax()))
    return seq[len(prompt):]
