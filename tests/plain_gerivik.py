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


def route_margin(h, w, pre, r):
    """How far every token's choice is from another one [T]: the smaller of the gap between the last kept and the
    first dropped group and the gap between the last chosen and the first unchosen output.  Tests leave out tokens
    whose margin is within rounding: there the choice is not the design's to decide."""
    s = torch.softmax(h @ w[pre + 'router'].t(), dim=-1)
    choice = s + w[pre + 'correction']
    total = r['experts'] + r['identity']
    count, keep = r['groups']['count'], r['groups']['keep']
    best = choice.reshape(-1, count, total // count).max(dim=-1).values
    margin = torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    if keep < count:
        ordered = best.sort(dim=-1, descending=True).values
        margin = ordered[:, keep - 1] - ordered[:, keep]
    kept = torch.zeros_like(best, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    ordered = choice.masked_fill(~kept.repeat_interleave(total // count, dim=1), -math.inf).sort(dim=-1, descending=True).values
    if r['top'] < total:
        margin = torch.minimum(margin, ordered[:, r['top'] - 1] - ordered[:, r['top']])
    return margin


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
def logits(tokens, weights, config, dtype=torch.float64, streams=None, margins=None):
    """Logits [T, vocab] of one sequence.  ``streams``: a list that receives the residual stream after every layer run;
    ``margins``: a list that receives every routed feed-forward's ``route_margin``."""
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
            if margins is not None:
                margins.append(route_margin(rms_norm(x, w[pre + 'norm2'], eps), w, pre + 'mlp.', layer['mlp']['router']))
            fed = moe(rms_norm(x, w[pre + 'norm2'], eps), w, pre + 'mlp.', layer['mlp'])
            x = x + rms_norm(fed, w[pre + 'norm2b'], eps)
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, w['final.norm'], eps) @ w['head'].t()


def greedy(prompt, count, weights, config, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(logits(tokens, weights, config, dtype)[-1].argmax()))
    return tokens[len(prompt):]


# ---------------------------------------------------------------------------------------------- configurations
def moe_mlp(*, ff, limit, experts, identity, top, count=1, keep=1):
    return dict(kind='moe', expert=dict(ff=ff, limit=limit),
                router=dict(experts=experts, identity=identity, top=top, groups=dict(count=count, keep=keep)))


def attention_layer(*, heads, kv_heads, dim, vdim, rot_dims, scale, softcap, base=10000.0, mlp=None):
    return dict(type='attention', mlp=mlp,
                mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot=dict(base=base, dims=rot_dims), scale=scale,
                           softcap=softcap))


def gla_layer(*, heads, dim, vdim, tau, mlp=None):
    return dict(type='gla', mlp=mlp, mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau))


def shared(config_layers, source):
    """One more run of layer ``source`` with a cache of its own."""
    return dict(config_layers[source], weights_of=source)


def make_config(layers, *, vocab, width, scale=1.0, eps=1e-6):
    return dict(architecture='Gerivik', vocab=vocab, width=width, embedding=dict(scale=scale), layers=layers,
                norm=dict(eps=eps))


def random_weights(config, seed, spread=1.0, decay_rank=5, decay_bias=2.0):
    """Tensors under the checkpoint's names, rounded to bfloat16 values (a float32 and a bfloat16 engine then read the
    same numbers).  ``spread`` scales the matrices around 1 / sqrt(fan-in); the decays' biases are shifted up so that
    the memories keep what they hold for tens of tokens."""
    g = torch.Generator().manual_seed(seed)
    width = config['width']

    def matrix(rows, columns, gain=1.0):
        return (torch.randn(rows, columns, generator=g) * (spread * gain / math.sqrt(columns))).to(torch.bfloat16).to(torch.float64)

    def scale(size):
        return (1.0 + 0.1 * torch.randn(size, generator=g)).to(torch.bfloat16).to(torch.float64)

    w = {'embed': matrix(config['vocab'], width, math.sqrt(width)), 'final.norm': scale(width), 'head': matrix(config['vocab'], width)}
    for index, layer in enumerate(config['layers']):
        if 'weights_of' in layer:
            continue
        pre, m = f'l{index}.', layer['mixer']
        w[pre + 'norm1'], w[pre + 'norm1b'] = scale(width), scale(width)
        if layer['type'] == 'attention':
            w[pre + 'mix.q'] = matrix(m['heads'] * m['dim'], width, 2.0)
            w[pre + 'mix.k'] = matrix(m['kv_heads'] * m['dim'], width, 2.0)
            w[pre + 'mix.v'] = matrix(m['kv_heads'] * m['vdim'], width)
            w[pre + 'mix.o'] = matrix(width, m['heads'] * m['vdim'])
        else:
            hd, hv = m['heads'] * m['dim'], m['heads'] * m['vdim']
            for name, rows in (('q', hd), ('k', hd), ('v', hv), ('g', hv)):
                w[pre + 'mix.' + name] = matrix(rows, width)
            w[pre + 'mix.o'] = matrix(width, hv)
            w[pre + 'mix.norm'] = scale(m['vdim'])
            w[pre + 'mix.a1'] = matrix(decay_rank, width, 2.0)
            w[pre + 'mix.a2'] = matrix(hd, decay_rank, 2.0)
            w[pre + 'mix.a2.b'] = (decay_bias + torch.randn(hd, generator=g)).to(torch.bfloat16).to(torch.float64)
        f = layer['mlp']
        if f is not None:
            r = f['router']
            w[pre + 'norm2'], w[pre + 'norm2b'] = scale(width), scale(width)
            w[pre + 'mlp.router'] = matrix(r['experts'] + r['identity'], width, 3.0)
            w[pre + 'mlp.correction'] = (0.2 * torch.randn(r['experts'] + r['identity'], generator=g)).to(torch.bfloat16).to(torch.float64)
            for e in range(r['experts']):
                w[f'{pre}mlp.e{e}.gate'] = matrix(f['expert']['ff'], width, 1.5)
                w[f'{pre}mlp.e{e}.up'] = matrix(f['expert']['ff'], width, 1.5)
                w[f'{pre}mlp.e{e}.down'] = matrix(width, f['expert']['ff'])
    return w
