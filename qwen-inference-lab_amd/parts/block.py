"""Pre-norm residual arrangement: norm -> sub-layer -> add to the un-normalised stream.

Two sub-layers per block, mixer then feed-forward (qil/model.py:48-71), or the mixer alone (``ffn=None``).  The
stream is float32 and every residual sum is made in float32; the add of a
sub-layer's output is fused into the norm that follows it.  ``residual_scale`` m: x + m * sublayer(norm(x)); the
norms multiply what they add, and the model multiplies the last block's output (``CausalLM(residual_scale=)``).
"""
from .base import Block
from .. import ops


class PreNormBlock(Block):
    def __init__(self, *, mixer_norm, mixer, ffn_norm=None, ffn=None, dtype, names=None, residual_scale=1.0):
        super().__init__()
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.dtype = mixer_norm, mixer, ffn_norm, ffn, dtype
        if (ffn is None) != (ffn_norm is None):
            raise ValueError('a feed-forward and its norm come together')
        self.residual_scale = float(residual_scale)
        self._names = names or dict(mixer_norm='mixer_norm', mixer='mixer', ffn_norm='ffn_norm', ffn='ffn')

    def parts(self):
        n = self._names
        out = {n['mixer_norm']: self.mixer_norm, n['mixer']: self.mixer}
        if self.ffn is not None:
            out.update({n['ffn_norm']: self.ffn_norm, n['ffn']: self.ffn})
        return out

    def forward(self, stream, pending, ctx, cache):
        if self.residual_scale != 1.0:
            return self._forward_scaled(stream, pending, ctx, cache)
        h = None
        if isinstance(pending, ops.Added):                     # the stream is complete
            if self.mixer.takes_lazy_norm:                     # the mixer's first product may make the norm itself
                h = self.mixer_norm.forward_lazy(stream, self.dtype, pending)
            pending = None
        if h is None:
            h = self.mixer_norm.forward(stream, pending, self.dtype)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return mixed
        h = self.ffn_norm.forward(stream, None if isinstance(mixed, ops.Added) else mixed, self.dtype)
        return self.ffn.forward(h, add_to=stream) if self.ffn.adds_to_stream else self.ffn.forward(h)

    def _forward_scaled(self, stream, pending, ctx, cache):
        """The same with every sub-layer output multiplied as it is added: nothing adds into the stream by itself."""
        m = self.residual_scale
        if isinstance(pending, ops.Added):
            pending = None
        h = self.mixer_norm.forward(stream, pending, self.dtype, delta_scale=m)
        mixed = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return mixed
        return self.ffn.forward(self.ffn_norm.forward(stream, mixed, self.dtype, delta_scale=m))


class SandwichBlock(Block):
    """A norm before and a norm after every sub-layer: x <- x + post(sublayer(pre(x))), mixer then feed-forward (or
    the mixer alone).  The stream and both norms' statistics are float32; a sub-layer's output leaves the block as an
    ``ops.PostNormed`` (not yet normed, not yet added), and the norm that follows, this block's or the next one's or
    the model's last, makes the post norm, the sum and its own norm in one kernel."""

    def __init__(self, *, mixer_norm, mixer, mixer_post_norm, ffn_norm=None, ffn=None, ffn_post_norm=None, dtype, names=None):
        super().__init__()
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm, self.dtype = ffn_norm, ffn, ffn_post_norm, dtype
        if len({ffn is None, ffn_norm is None, ffn_post_norm is None}) != 1:
            raise ValueError('a feed-forward and its two norms come together')
        self._names = names or dict(mixer_norm='mixer_norm', mixer='mixer', mixer_post_norm='mixer_post_norm',
                                    ffn_norm='ffn_norm', ffn='ffn', ffn_post_norm='ffn_post_norm')

    def parts(self):
        n = self._names
        out = {n['mixer_norm']: self.mixer_norm, n['mixer']: self.mixer, n['mixer_post_norm']: self.mixer_post_norm}
        if self.ffn is not None:
            out.update({n['ffn_norm']: self.ffn_norm, n['ffn']: self.ffn, n['ffn_post_norm']: self.ffn_post_norm})
        return out

    @staticmethod
    def _post(norm, value):
        return ops.PostNormed(value, norm.p['weight'], norm.eps)

    def forward(self, stream, pending, ctx, cache):
        if isinstance(pending, ops.Added):                     # the stream is complete
            pending = None
        h = self.mixer_norm.forward(stream, pending, self.dtype)
        mixed = self._post(self.mixer_post_norm, self.mixer.forward(h, ctx, cache))
        if self.ffn is None:
            return mixed
        h = self.ffn_norm.forward(stream, mixed, self.dtype)
        return self._post(self.ffn_post_norm, self.ffn.forward(h))
