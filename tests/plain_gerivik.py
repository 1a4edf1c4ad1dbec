"""A plain, slow restatement of the Gerivik design: one function per mechanism, whole sequences, no cache.

Test code only: it shares nothing with the engine.  Everything runs in one dtype (float64 by default) on the CPU.
Weights are a dict name -> tensor under the checkpoint's own names; ``config`` is the config.json dict.

Notation: x [T, width] is the residual stream of one sequence, h a sub-layer's input, H heads, G key/value heads.
"""
import math

import torch

SWISH_SLOPE = 1.702


# ---------------------------------------------------------------------------------------------- small pieces
def rms_unit(x, eps):
    return x / torch.sqrt(x.square().mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def rotate_half(x, positions, base, dims):
    """Rotate the first ``dims`` elements of the last axis; element i pairs with i + dims / 2.  x [T, heads, d]."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


# ---------------------------------------------------------------------------------------------- mixers
def attention(h, w, pre, m, eps, positions):
    """Grouped-query attention: partly rotated queries and keys, brought to unit root mean square per head after the
    rotation, scores scaled and then soft-capped, a causal softmax."""
    t = h.shape[0]
    heads, groups, d, dv = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    q = (h @ w[pre + 'q'].t()).reshape(t, heads, d)
    k = (h @ w[pre + 'k'].t()).reshape(t, groups, d)
    v = (h @ w[pre + 'v'].t()).reshape(t, groups, dv)
    q = rms_unit(rotate_half(q, positions, m['rot']['base'], m['rot']['dims']), eps)
    k = rms_unit(rotate_half(k, positions, m['rot']['base'], m['rot']['dims']), eps)
    share = heads // groups
    k = k.repeat_interleave(share, dim=1)                        # query head a reads key/value head a // share
    v = v.repeat_interleave(share, dim=1)
    scores = torch.einsum('ihd,jhd->hij', q, k) * m['scale']
    scores = m['softcap'] * torch.tanh(scores / m['softcap'])
    visible = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~visible[None], -math.inf)
    out = torch.einsum('hij,jhd->ihd', torch.softmax(scores, dim=-1), v).reshape(t, heads * dv)
    return out @ w[pre + 'o'].t()


def gla(h, w, pre, m, eps):
    """Gated linear attention: a [dim, vdim] memory per head whose rows (key channels) each decay by a factor of their
    own, made from the input through a low-rank product."""
    t = h.shape[0]
    heads, d, dv = m['heads'], m['dim'], m['vdim']
    q = (h @ w[pre + 'q'].t()).reshape(t, heads, d) * d ** -0.5
    k = (h @ w[pre + 'k'].t()).reshape(t, heads, d)
    v = (h @ w[pre + 'v'].t()).reshape(t, heads, dv)
    z = (h @ w[pre + 'a1'].t()) @ w[pre + 'a2'].t() + w[pre + 'a2.b']
    keep = torch.sigmoid(z).pow(1.0 / m['tau']).reshape(t, heads, d)
    memory = torch.zeros(heads, d, dv, dtype=h.dtype)
    outs = []
    for i in range(t):
        memory = keep[i][:, :, None] * memory + k[i][:, :, None] * v[i][:, None, :]
        outs.append(torch.einsum('hdv,hd->hv', memory, q[i]))
    o = rms_norm(torch.stack(outs), w[pre + 'norm'], eps).reshape(t, heads * dv)
    gate = h @ w[pre + 'g'].t()
    return (o * gate * torch.sigmoid(gate)) @ w[pre + 'o'].t()


# ---------------------------------------------------------------------------------------------- feed-forward
def expert(h, w, pre, limit):
    g = (h @ w[pre + 'gate'].t()).clamp(max=limit)
    u = (h @ w[pre + 'up'].t()).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(SWISH_SLOPE * g) * (u + 1)) @ w[pre + 'down'].t()


def route(h, w, pre, r):
    """(chosen [T, top] indices, weights [T, top]) over experts + identity outputs."""
    s = torch.softmax(h @ w[pre + 'router'].t(), dim=-1)
    choice = s + w[pre + 'correction']
    total = r['experts'] + r['identity']
    count, keep = r['groups']['count'], r['groups']['keep']
    best = choice.reshape(-1, count, total // count).max(dim=-1).values              # [T, groups]
    kept = torch.zeros_like(best, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    choice = choice.masked_fill(~kept.repeat_interleave(total // count, dim=1), -math.inf)
    chosen = choice.topk(r['top'], dim=-1).indices
    return chosen, s.gather(1, chosen)


def moe(h, w, pre, f):
    r = f['router']
    chosen, weights = route(h, w, pre, r)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, weight in zip(chosen[i].tolist(), weights[i]):
            if e >= r['experts']:                                                      # an identity expert
                out[i] += weight * h[i]
            else:
                out[i] += weight * expert(h[i:i + 1], w, f'{pre}e{e}.', f['expert']['limit'])[0]
    return out


# ---------------------------------------------------------------------------------------------- the model
def logits(tokens, weights, config, dtype=torch.float64, streams=None):
    """Logits [T, vocab] of one sequence.  ``streams``: a list that receives the residual stream after every layer run."""
    w = {name: t.to(dtype) for name, t in weights.items()}
    eps = config['norm']['eps']
    positions = torch.arange(len(tokens))
    x = w['embed'][torch.tensor(tokens)] * config['embedding']['scale']
    for index, layer in enumerate(config['layers']):
        pre = f"l{layer.get('weights_of', index)}."
        h = rms_norm(x, w[pre + 'norm1'], eps)
        if layer['type'] == 'attention':
            mixed = attention(h, w, pre + 'mix.', layer['mixer'], eps, positions)
        else:
            mixed = gla(h, w, pre + 'mix.', layer['mixer'], eps)
        x = x + rms_norm(mixed, w[pre + 'norm1b'], eps)
        if layer['mlp'] is not None:
            fed = moe(rms_norm(x, w[pre + 'norm2'], eps), w, pre + 'mlp.', layer['mlp'])
            x = x + rms_norm(fed, w[pre + 'norm2b'], eps)
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, w['final.norm'], eps) @ w['head'].t()
