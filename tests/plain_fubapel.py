"""A plain, slow restatement of the Fubapel design: one function per mechanism, whole sequences, no cache.

Test code only: it shares nothing with the engine.  Everything runs in one dtype (float64 by default) on the CPU.
Weights are a dict name -> tensor under the checkpoint's own names; ``config`` is the config.json dict.

Notation: x [T, width] is the residual stream of one sequence, h a sub-layer's input, H heads.
"""
import math

import torch


# ---------------------------------------------------------------------------------------------- small pieces
def layer_norm(x, weight, eps):
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(centred.square().mean(dim=-1, keepdim=True) + eps) * weight


def rms_unit(x, eps):
    return x / torch.sqrt(x.square().mean(dim=-1, keepdim=True) + eps)


def rotate_half(x, positions, base, dims):
    """Rotate the first ``dims`` elements of the last axis; element i pairs with i + dims / 2.  x [T, ..., d]."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = angle.cos().reshape(shape), angle.sin().reshape(shape)
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def log_sigmoid(z):
    return -torch.nn.functional.softplus(-z)


# ---------------------------------------------------------------------------------------------- mixers
def latent_attention(h, w, pre, m, eps, positions):
    """Attention whose keys and values are expanded from one low-rank latent per token, one rotated key part shared
    by all heads, and a per-head sink logit in the softmax's denominator."""
    t = h.shape[0]
    heads, d, r, dv, rank = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank']
    cq = rms_unit(h @ w[pre + 'dq'].t(), eps) * w[pre + 'dq.norm']
    q = (cq @ w[pre + 'uq'].t()).reshape(t, heads, d + r)
    q_plain, q_rot = q[..., :d], rotate_half(q[..., d:], positions, m['rot']['base'], m['rot']['dims'])
    down = h @ w[pre + 'dkv'].t()
    c = rms_unit(down[:, :rank], eps) * w[pre + 'dkv.norm']
    k_rot = rotate_half(down[:, rank:], positions, m['rot']['base'], m['rot']['dims'])           # [T, r], every head's
    k_plain = (c @ w[pre + 'uk'].t()).reshape(t, heads, d)
    v = (c @ w[pre + 'uv'].t()).reshape(t, heads, dv)
    scores = (torch.einsum('ihd,jhd->hij', q_plain, k_plain) + torch.einsum('ihr,jr->hij', q_rot, k_rot)) * m['scale']
    visible = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~visible[None], -math.inf)
    sink = w[pre + 'sink'].to(h.dtype)                                                          # [H]
    top = torch.maximum(scores.max(dim=-1).values, sink[:, None])                               # [H, T]
    e = torch.exp(scores - top[..., None])
    p = e / (e.sum(dim=-1) + torch.exp(sink[:, None] - top))[..., None]
    out = torch.einsum('hij,jhv->ihv', p, v).reshape(t, heads * dv)
    return out @ w[pre + 'o'].t()


def mlstm(h, w, pre, m, eps):
    """Matrix memory with exponential input gate, stabilised by a running maximum that starts at 0."""
    t = h.shape[0]
    heads, d, dv, cap = m['heads'], m['dim'], m['vdim'], m['gate_cap']
    q = (h @ w[pre + 'q'].t()).reshape(t, heads, d) * d ** -0.5
    k = (h @ w[pre + 'k'].t()).reshape(t, heads, d)
    v = (h @ w[pre + 'v'].t()).reshape(t, heads, dv)
    log_in = cap * torch.tanh((h @ w[pre + 'i'].t() + w[pre + 'i.b']) / cap)                     # [T, H]
    log_keep = log_sigmoid(cap * torch.tanh((h @ w[pre + 'f'].t() + w[pre + 'f.b']) / cap))
    memory = torch.zeros(heads, d, dv, dtype=h.dtype)
    norm = torch.zeros(heads, d, dtype=h.dtype)
    top = torch.zeros(heads, dtype=h.dtype)
    out = torch.zeros(t, heads, dv, dtype=h.dtype)
    for step in range(t):
        new_top = torch.maximum(log_keep[step] + top, log_in[step])
        keep, take = torch.exp(log_keep[step] + top - new_top), torch.exp(log_in[step] - new_top)
        memory = keep[:, None, None] * memory + take[:, None, None] * k[step][:, :, None] * v[step][:, None, :]
        norm = keep[:, None] * norm + take[:, None] * k[step]
        top = new_top
        read = torch.einsum('hdv,hd->hv', memory, q[step])
        below = torch.maximum((norm * q[step]).sum(dim=-1).abs(), torch.exp(-top)) + 1e-6
        out[step] = read / below[:, None]
    out = rms_unit(out, eps).reshape(t, heads * dv) * w[pre + 'norm']
    return (out * torch.sigmoid(h @ w[pre + 'g'].t())) @ w[pre + 'o'].t()


def retention(h, w, pre, m, eps, positions):
    """Linear attention with a fixed decay per head; no softmax, no denominator."""
    t = h.shape[0]
    heads, d, dv = m['heads'], m['dim'], m['vdim']
    q = rotate_half((h @ w[pre + 'q'].t()).reshape(t, heads, d), positions, m['rot']['base'], m['rot']['dims'])
    k = rotate_half((h @ w[pre + 'k'].t()).reshape(t, heads, d), positions, m['rot']['base'], m['rot']['dims']) * d ** -0.5
    v = (h @ w[pre + 'v'].t()).reshape(t, heads, dv)
    decay = torch.tensor(m['decay'], dtype=h.dtype)
    memory = torch.zeros(heads, d, dv, dtype=h.dtype)
    out = torch.zeros(t, heads, dv, dtype=h.dtype)
    for step in range(t):
        memory = decay[:, None, None] * memory + k[step][:, :, None] * v[step][:, None, :]
        out[step] = torch.einsum('hdv,hd->hv', memory, q[step])
    out = rms_unit(out, eps).reshape(t, heads * dv)
    gate = h @ w[pre + 'g'].t()
    return (out * gate * torch.sigmoid(gate)) @ w[pre + 'o'].t()


def dense_ff(h, w, pre, f):
    gate = torch.clamp(h @ w[pre + 'gate'].t(), max=f['limit'])
    up = torch.clamp(h @ w[pre + 'up'].t(), min=-f['limit'], max=f['limit'])
    return (gate * torch.sigmoid(1.702 * gate) * (up + 1)) @ w[pre + 'down'].t()


MIXERS = {
    'latent_attention': lambda h, w, pre, m, eps, pos: latent_attention(h, w, pre, m, eps, pos),
    'mlstm': lambda h, w, pre, m, eps, pos: mlstm(h, w, pre, m, eps),
    'retention': lambda h, w, pre, m, eps, pos: retention(h, w, pre, m, eps, pos),
}


# ---------------------------------------------------------------------------------------------- the model
def layer_order(config):
    """Indices of the layers in the order they run: the looped span repeated, then the rest."""
    count = len(config['layers'])
    loop = config.get('loop') or dict(start=0, stop=0, times=1)
    span = list(range(loop['start'], loop['stop']))
    return list(range(loop['start'])) + span * loop['times'] + list(range(loop['stop'], count))


def run_layer(x, w, config, index, positions):
    spec, eps, mult = config['layers'][index], config['norm']['eps'], config['residual_mult']
    pre = f'l{index}.'
    x = x + mult * MIXERS[spec['type']](layer_norm(x, w[pre + 'norm1'], eps), w, pre + 'mix.', spec['mixer'], eps, positions)
    if spec.get('mlp') is not None:
        x = x + mult * dense_ff(layer_norm(x, w[pre + 'norm2'], eps), w, pre + 'mlp.', spec['mlp'])
    return x


def logits(tokens, w, config, dtype=torch.float64, streams=None):
    """[T, vocab] for one whole sequence.  ``streams``: a list that receives the residual stream after every layer run."""
    w = {name: t.to(dtype) if t.is_floating_point() else t for name, t in w.items()}
    positions = torch.arange(len(tokens))
    x = w['embed'][torch.as_tensor(tokens)]
    for index in layer_order(config):
        x = run_layer(x, w, config, index, positions)
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, w['final.norm'], config['norm']['eps']) @ w['head'].t()


def greedy(prompt, new_tokens, w, config, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(logits(tokens, w, config, dtype)[-1].argmax()))
    return tokens[len(prompt):]


# ---------------------------------------------------------------------------------------------- random models
def tensor_shapes(config):
    """name -> (shape, kind) of every tensor of a configuration; kind: matrix | scale | bias | sink."""
    width, out = config['width'], {}
    out['embed'] = ((config['vocab'], width), 'matrix')
    for index, spec in enumerate(config['layers']):
        pre, m = f'l{index}.', spec['mixer']
        out[pre + 'norm1'] = ((width,), 'scale')
        if spec['type'] == 'latent_attention':
            heads, d, r, dv = m['heads'], m['dim'], m['rot_dim'], m['vdim']
            out[pre + 'mix.dq'] = ((m['q_rank'], width), 'matrix')
            out[pre + 'mix.dq.norm'] = ((m['q_rank'],), 'scale')
            out[pre + 'mix.uq'] = ((heads * (d + r), m['q_rank']), 'matrix')
            out[pre + 'mix.dkv'] = ((m['kv_rank'] + r, width), 'matrix')
            out[pre + 'mix.dkv.norm'] = ((m['kv_rank'],), 'scale')
            out[pre + 'mix.uk'] = ((heads * d, m['kv_rank']), 'matrix')
            out[pre + 'mix.uv'] = ((heads * dv, m['kv_rank']), 'matrix')
            out[pre + 'mix.sink'] = ((heads,), 'sink')
            out[pre + 'mix.o'] = ((width, heads * dv), 'matrix')
        else:
            heads, d, dv = m['heads'], m['dim'], m['vdim']
            for name, rows in (('q', heads * d), ('k', heads * d), ('v', heads * dv), ('g', heads * dv)):
                out[pre + 'mix.' + name] = ((rows, width), 'matrix')
            out[pre + 'mix.o'] = ((width, heads * dv), 'matrix')
            if spec['type'] == 'mlstm':
                out[pre + 'mix.norm'] = ((heads * dv,), 'scale')
                for gate in ('i', 'f'):
                    out[pre + f'mix.{gate}'] = ((heads, width), 'matrix')
                    out[pre + f'mix.{gate}.b'] = ((heads,), 'bias')
        if spec.get('mlp') is not None:
            out[pre + 'norm2'] = ((width,), 'scale')
            out[pre + 'mlp.gate'] = ((spec['mlp']['ff'], width), 'matrix')
            out[pre + 'mlp.up'] = ((spec['mlp']['ff'], width), 'matrix')
            out[pre + 'mlp.down'] = ((width, spec['mlp']['ff']), 'matrix')
    out['final.norm'] = ((width,), 'scale')
    out['head'] = ((config['vocab'], width), 'matrix')
    return out


def random_weights(config, seed, spread=1.0):
    """Weights rounded to bfloat16 (so that a bfloat16 and a float32 engine read the same values), held as float32.
    Matrices N(0, spread / fan_in); scales 1 + N(0, 0.1); gate biases and sinks N(0, 1)."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, (shape, kind) in tensor_shapes(config).items():
        noise = torch.randn(shape, generator=g)
        if kind == 'matrix':
            value = noise * (spread / shape[-1]) ** 0.5 if name != 'embed' else noise
        elif kind == 'scale':
            value = 1 + 0.1 * noise
        else:
            value = noise
        w[name] = value.to(torch.bfloat16).to(torch.float32)
    return w


def attention_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=24, base=10000.0, ff=None, limit=2.0):
    return dict(type='latent_attention',
                mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
                           rot=dict(base=base, dims=rot_dim), scale=(dim + rot_dim) ** -0.5),
                mlp=None if ff is None else dict(kind='dense', ff=ff, limit=limit))


def mlstm_layer(heads=2, dim=24, vdim=16, gate_cap=15.0, ff=None, limit=2.0):
    return dict(type='mlstm', mixer=dict(heads=heads, dim=dim, vdim=vdim, gate_cap=gate_cap),
                mlp=None if ff is None else dict(kind='dense', ff=ff, limit=limit))


def retention_layer(heads=3, dim=16, vdim=24, decay=(0.9, 0.97, 0.995), base=5000.0, rot_dims=None, ff=None, limit=2.0):
    return dict(type='retention', mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay),
                                             rot=dict(base=base, dims=dim if rot_dims is None else rot_dims)),
                mlp=None if ff is None else dict(kind='dense', ff=ff, limit=limit))


def make_config(layers, *, vocab=97, width=48, loop=None, eps=1e-5, residual_mult=0.8):
    return dict(architecture='Fubapel', vocab=vocab, width=width, layers=list(layers),
                loop=loop or dict(start=0, stop=0, times=1), norm=dict(eps=eps), residual_mult=residual_mult)
