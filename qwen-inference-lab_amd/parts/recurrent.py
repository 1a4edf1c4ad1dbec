"""Mixers with a matrix memory per head, carried from token to token in a state slot."""
import torch

from .base import Mixer, ParamSpec, StateNeed
from .. import ops


class MatrixMemory(Mixer):
    """Per head a state S [dim, vdim] in float32:  S_t = a_t S_(t-1) + b_t k_t v_t^T,  o_t = S_t^T q_t, then per head
    o / rms(o) (times ``out_norm`` weights over all heads if asked), times a gate act(W_g x), then W_o.

    ``gating='decay'``   a_t = decay[h] (constants of the configuration), b_t = 1; no denominator.
    ``gating='mlstm'``   exponential input gate and sigmoid forget gate in log space, both soft-capped:
                         i_t = cap tanh((W_i x + b_i) / cap),  f_t = logsigmoid(cap tanh((W_f x + b_f) / cap)),
                         m_t = max(f_t + m_(t-1), i_t) with m = 0 at the start, a_t = exp(f_t + m_(t-1) - m_t),
                         b_t = exp(i_t - m_t), n_t = a_t n_(t-1) + b_t k_t,
                         o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
    ``gating='channel'`` a decay per row i of S (key channel) and token: a_t[i] = sigmoid(z_t[i])^(1 / tau) with
                         z_t = W_up (W_down x) + b_up over all heads' rows (a low-rank product whose inner size the
                         checkpoint decides; ``decay_rank`` is what random weights get), b_t = 1; no denominator.
    ``out_norm``         True: the head norm has weights; ``out_norm_shared``: one weight [vdim] for all heads.
    ``position``         a ``RotaryFrequencies`` or None: queries and keys are rotated on their leading rot_dim elements.
    ``q_scale``, ``k_scale`` multiply queries and keys after the rotation.  ``gate``: 'sigmoid' or 'silu'.

    The recurrence, the gates, the rotation and the head norm are float32; the projections are the model's type, the
    gate pre-activations of 'mlstm' come out of their product in float32.
    """
    graph_safe = True

    def __init__(self, *, width, heads, dim, vdim, gating, eps, gate, out_norm=False, decay=None, cap=None,
                 position=None, q_scale=1.0, k_scale=1.0, dtype=torch.bfloat16, tau=None, decay_rank=16,
                 out_norm_shared=False):
        super().__init__()
        for name, value in (('heads', heads), ('dim', dim), ('vdim', vdim)):
            if type(value) is not int or value < 1:
                raise ops.UnsupportedShape(f'{name} must be a positive integer, not {value!r}')
        if gating not in ops.SCAN_MODES or gate not in ('sigmoid', 'silu'):
            raise ValueError(f'unknown gating {gating!r} or gate {gate!r}')
        if gating == 'decay' and (decay is None or len(decay) != heads):
            raise ValueError('one decay per head')
        if gating == 'mlstm' and not (cap is not None and cap > 0):
            raise ValueError('the gates need a positive cap')
        if gating == 'channel' and not (tau is not None and tau > 0):
            raise ValueError('the decays need a positive tau')
        self.tau, self.decay_rank, self.out_norm_shared = float(tau or 0.0), int(decay_rank), bool(out_norm_shared)
        self.rot = position.rot_dim if position is not None else 0
        if self.rot > dim or dim > 256:
            raise ops.UnsupportedShape(f'dim {dim}: the recurrence kernel takes up to 256, rotated elements up to dim')
        self.width, self.heads, self.dim, self.vdim, self.gating = width, heads, dim, vdim, gating
        self.eps, self.gate, self.out_norm, self.cap = float(eps), gate, bool(out_norm), float(cap or 0.0)
        self.decay_values = None if decay is None else [float(x) for x in decay]
        self.position, self.q_scale, self.k_scale, self.dtype = position, float(q_scale), float(k_scale), dtype
        self._decay = None

    def param_specs(self):
        h, d, v = self.heads, self.dim, self.vdim
        specs = {'q_proj.weight': ParamSpec((h * d, self.width)), 'k_proj.weight': ParamSpec((h * d, self.width)),
                 'v_proj.weight': ParamSpec((h * v, self.width)), 'g_proj.weight': ParamSpec((h * v, self.width)),
                 'o_proj.weight': ParamSpec((self.width, h * v))}
        if self.out_norm:
            specs['out_norm.weight'] = ParamSpec((v if self.out_norm_shared else h * v,), 'vector', 'one_plus_normal')
        if self.gating == 'channel':
            specs.update({'decay_down.weight': ParamSpec((self.decay_rank, self.width), free=(0,)),
                          'decay_up.weight': ParamSpec((h * d, self.decay_rank), free=(1,)),
                          'decay_up.bias': ParamSpec((h * d,), 'vector')})
        if self.gating == 'mlstm':
            specs.update({'i_gate.weight': ParamSpec((h, self.width)), 'i_gate.bias': ParamSpec((h,), 'vector'),
                          'f_gate.weight': ParamSpec((h, self.width)), 'f_gate.bias': ParamSpec((h,), 'vector')})
        return specs

    def cache_need(self):
        return StateNeed((ops.state_scan_slot(heads=self.heads, dim=self.dim, vdim=self.vdim, mode=self.gating),), 'float32')

    def finalize(self):
        p = self.p
        self.w_in = torch.cat([p.pop(name) for name in ('q_proj.weight', 'k_proj.weight', 'v_proj.weight',
                                                        'g_proj.weight')]).contiguous()
        p['in_proj.weight'] = self.w_in
        if self.out_norm and self.out_norm_shared:
            p['out_norm.weight'] = p['out_norm.weight'].repeat(self.heads).contiguous()      # a pure re-layout
        if self.gating == 'mlstm':
            p['gates.weight'] = torch.cat([p.pop('i_gate.weight'), p.pop('f_gate.weight')]).contiguous()
            p['gates.bias'] = torch.cat([p.pop('i_gate.bias'), p.pop('f_gate.bias')]).contiguous()
        elif self.gating == 'channel':
            if p['decay_down.weight'].shape[0] != p['decay_up.weight'].shape[1]:
                raise ValueError(f"the decay's two matrices do not fit: {tuple(p['decay_down.weight'].shape)} and "
                                 f"{tuple(p['decay_up.weight'].shape)}")
        else:                                           # device tensors are made here, not in a step that may be captured
            self._decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(self.w_in.device)
        if self.position is not None:
            self.position.frequencies()

    def forward(self, h, ctx, cache):
        p = self.p
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        proj = ops.linear(h, self.w_in, None)
        extra = {}
        if self.gating == 'mlstm':
            extra = dict(gates=ops.linear(h, p['gates.weight'], None, out_dtype=torch.float32), gate_bias=p['gates.bias'],
                         cap=self.cap)
        elif self.gating == 'channel':                  # z in float32 out of the second product; the rest in the scan
            low = ops.linear(h, p['decay_down.weight'], None)
            extra = dict(gates=ops.linear(low, p['decay_up.weight'], p['decay_up.bias'], out_dtype=torch.float32),
                         cap=self.tau)
        else:
            extra = dict(decay=self._decay)
        if self.position is not None:
            extra.update(frequencies=self.position.frequencies(), rot=self.rot)
        raw, below = ops.state_scan(proj, mode=self.gating, heads=self.heads, dim=self.dim, vdim=self.vdim, q_offset=0,
                                    k_offset=hd, v_offset=2 * hd, state=cache.state, cu_seqlens=ctx.cu_seqlens,
                                    seq_starts=ctx.seq_starts, seq_slots=ctx.seq_slots, n_seqs=ctx.n_seqs,
                                    q_scale=self.q_scale, k_scale=self.k_scale, max_query=ctx.max_query, **extra)
        gated = ops.head_norm_gate(raw, proj, gate_offset=2 * hd + hv, heads=self.heads, vdim=self.vdim,
                                   weight=p.get('out_norm.weight'), eps=self.eps, gate=self.gate, out_dtype=self.dtype,
                                   denominators=below)
        return ops.linear(gated, p['o_proj.weight'], None, partials=True)
