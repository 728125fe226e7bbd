"""Arrangements: how one layer orders its norms, mixer, feed-forward and residual sums.

"prenorm":    x += mixer(norm(x));  x += ffn(norm(x))   (reference atomserve/model.py:378-382)
"two_norms":  x += mixer(norm1(x)) + ffn(norm2(x)), both parts reading the same x through a norm each
"gated_prenorm": x += m g1(h) * mixer(h), h = norm(x);  x += m g2(h) * ffn(h), h = norm(x), with sigmoid gates g

The residual stream `x` is fp32 in both precisions.  A part's output is not added at
once: it travels as the pending `delta` to the next norm, whose kernel adds it into
`x` and normalises in one pass.  With few rows (decoding) both steps move into the matrix
products around them instead: a part's last product adds into `x` and leaves the next norm
pending (`Norm.absorb`), and the next part's first product finishes it (`PendingNorm`).
"""

from atomserve_amd.parts.base import Arrangement, DeltaSum, GatedDelta, PendingNorm, build, register


class PreNormBlock(Arrangement):
    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = build("norm", spec.ffn_norm, env)
        self.ffn = build("feed_forward", spec.ffn, env)

    def parts(self) -> dict:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def first_norm(self):
        return self.mixer_norm

    def forward(self, x, delta, step, cache, next_norm=None):
        delta = self.apply(self.mixer_norm, self.mixer, self.ffn_norm, x, delta, step, cache)
        return self.apply(self.ffn_norm, self.ffn, next_norm, x, delta, step)

    @staticmethod
    def apply(norm, part, next_norm, x, delta, *args):
        """part(norm(x + delta)): the part's output still to be added, or the PendingNorm of
        `next_norm` if the part added it itself.  `delta` may be the PendingNorm of `norm`."""
        if isinstance(delta, PendingNorm):
            h = delta if part.takes_pending_norm else delta.rows()
        else:
            h = norm.forward(x, delta)
        if part.adds_to_residual:
            return part.forward(h, *args, residual=x, next_norm=next_norm)
        return part.forward(h, *args)


register("arrangement", "prenorm", PreNormBlock)


class TwoNormsBlock(Arrangement):
    """x += mixer(mixer_norm(x)) + ffn(ffn_norm(x)): the two parts read the same stream, each through a norm of
    its own.  Both outputs travel on as one pending `DeltaSum`; the kernel that starts the next layer adds them
    into the stream (in fp32) and takes both of that layer's norms from one root mean square.  A layer without
    a feed-forward (spec.ffn None) is the mixer alone."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        self.shared_kernel = self.ffn is not None and hasattr(self.mixer_norm, "with_sibling") and \
            type(self.mixer_norm) is type(self.ffn_norm) and spec.mixer_norm.eps == spec.ffn_norm.eps  # fmt: skip

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        return parts

    def first_norm(self):
        return None  # nothing is left pending inside a product for this layer: it takes a sum of outputs

    def forward(self, x, delta, step, cache, next_norm=None):
        if isinstance(delta, PendingNorm):
            raise ValueError("a layer of two norms takes pending outputs, not a norm left pending in a product")
        if self.shared_kernel:
            h1, h2 = self.mixer_norm.with_sibling(self.ffn_norm, x, delta)
        else:
            h1 = self.mixer_norm.forward(x, delta)
            h2 = self.ffn_norm.forward(x) if self.ffn is not None else None
        mixed = self.mixer.forward(h1, step, cache)
        if self.ffn is None:
            return mixed
        return DeltaSum((mixed, self.ffn.forward(h2, step)))


register("arrangement", "two_norms", TwoNormsBlock)


class GatedPreNormBlock(Arrangement):
    """x += m * sigmoid(G h + b) * part(h), h = norm(x), for the mixer and then for the feed-forward (spec.ffn
    None: the mixer alone); m = spec.residual_scale.  The gate reads what the part reads, so its logits are rows
    of the part's own input product (parts built with `out_gate` return a `GatedDelta`); the sigmoid, the
    product with the part's output and the sum into the fp32 stream happen in the kernel of the norm that follows."""

    def __init__(self, spec, env):
        super().__init__(spec, env)
        self.mixer_norm = build("norm", spec.mixer_norm, env)
        self.mixer = build("mixer", spec.mixer, env)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build("norm", spec.ffn_norm, env)
            self.ffn = build("feed_forward", spec.ffn, env)
        for name, part in (("mixer", spec.mixer), ("feed-forward", spec.ffn)):
            if part is not None and not getattr(part, "out_gate", False):
                raise ValueError(f"a layer with gated residual sums needs a {name} that computes its output gate (out_gate)")
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and not norm.takes_gated_delta:
                raise ValueError(f"a norm of kind {norm.spec.kind!r} does not add gated outputs into the stream")

    def parts(self) -> dict:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        return parts

    def first_norm(self):
        return None  # the layer before hands over its output, not a norm left pending in a product

    def forward(self, x, delta, step, cache, next_norm=None):
        if isinstance(delta, (PendingNorm, DeltaSum)):
            raise ValueError("a layer with gated residual sums takes a pending output, gated or plain")
        m = self.spec.residual_scale
        delta = self.mixer.forward(self.mixer_norm.forward(x, delta), step, cache).scaled(m)
        if self.ffn is None:
            return delta
        return self.ffn.forward(self.ffn_norm.forward(x, delta), step).scaled(m)


register("arrangement", "gated_prenorm", GatedPreNormBlock)
