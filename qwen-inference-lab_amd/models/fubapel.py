"""Fubapel assembled from parts.

Token embedding; layers of three kinds of mixer, chosen layer by layer by the configuration (attention over a cached
latent with a sink, an exponentially gated matrix memory, a matrix memory with fixed decays), each followed by a dense
gated feed-forward or by nothing; pre-norm with a layer norm (weight, no bias) and x + m * sublayer(norm(x)); a span
of layers may run several times in a row with the same weights, every run with a cache or state of its own; final
layer norm and an untied head.
"""
import torch

from ..config.fubapel import FubapelConfig
from ..parts import (LayerNorm, RotaryFrequencies, LatentAttention, MatrixMemory, GatedMLP, PreNormBlock, Embedding,
                     LMHead, CausalLM, ScheduleEntry)
from ..registry import register_architecture

SWISH_SLOPE = 1.702          # the slope inside the feed-forward gate's sigmoid: fixed by the design


def _latent_attention(width, m, eps, dtype, device):
    return LatentAttention(width=width, heads=m['heads'], dim=m['dim'], rot_dim=m['rot_dim'], vdim=m['vdim'],
                           kv_rank=m['kv_rank'], q_rank=m['q_rank'], scale=m['scale'], eps=eps, sink=True,
                           position=RotaryFrequencies(m['rot']['dims'], m['rot']['base'], device=device), dtype=dtype)


def _mlstm(width, m, eps, dtype, device):
    return MatrixMemory(width=width, heads=m['heads'], dim=m['dim'], vdim=m['vdim'], gating='mlstm', cap=m['gate_cap'],
                        eps=eps, gate='sigmoid', out_norm=True, q_scale=m['dim'] ** -0.5, dtype=dtype)


def _retention(width, m, eps, dtype, device):
    return MatrixMemory(width=width, heads=m['heads'], dim=m['dim'], vdim=m['vdim'], gating='decay', decay=m['decay'],
                        eps=eps, gate='silu', out_norm=False, k_scale=m['dim'] ** -0.5,
                        position=RotaryFrequencies(m['rot']['dims'], m['rot']['base'], device=device), dtype=dtype)


def _dense(width, f, dtype):
    return GatedMLP(width=width, intermediate=f['ff'], activation='clamped_swish', limit=f['limit'], alpha=SWISH_SLOPE,
                    dtype=dtype)


MIXERS = {'latent_attention': _latent_attention, 'mlstm': _mlstm, 'retention': _retention}
FEED_FORWARDS = {'dense': _dense}

# checkpoint suffix -> the part's own tensor name
_MIXER_TENSORS = {
    'latent_attention': {'dq': 'q_down.weight', 'dq.norm': 'q_norm.weight', 'uq': 'q_up.weight', 'dkv': 'kv_down.weight',
                         'dkv.norm': 'kv_norm.weight', 'uk': 'k_up.weight', 'uv': 'v_up.weight', 'sink': 'sink',
                         'o': 'o_proj.weight'},
    'mlstm': {'q': 'q_proj.weight', 'k': 'k_proj.weight', 'v': 'v_proj.weight', 'g': 'g_proj.weight', 'o': 'o_proj.weight',
              'norm': 'out_norm.weight', 'i': 'i_gate.weight', 'i.b': 'i_gate.bias', 'f': 'f_gate.weight',
              'f.b': 'f_gate.bias'},
    'retention': {'q': 'q_proj.weight', 'k': 'k_proj.weight', 'v': 'v_proj.weight', 'g': 'g_proj.weight',
                  'o': 'o_proj.weight'},
}
_FFN_TENSORS = {'gate': 'gate_proj.weight', 'up': 'up_proj.weight', 'down': 'down_proj.weight'}


def build_fubapel(config, *, dtype=torch.bfloat16, device='cuda'):
    width, eps = config.width, config.norm_eps
    embedding = Embedding(config.vocab, width)
    blocks, names = [], {'embed': (embedding, 'weight')}
    for index, layer in enumerate(config.layers):
        mixer = MIXERS[layer['type']](width, layer['mixer'], eps, dtype, device)
        ffn = FEED_FORWARDS[layer['mlp']['kind']](width, layer['mlp'], dtype) if layer['mlp'] is not None else None
        block = PreNormBlock(mixer_norm=LayerNorm(width, eps), mixer=mixer,
                             ffn_norm=LayerNorm(width, eps) if ffn is not None else None, ffn=ffn, dtype=dtype,
                             residual_scale=config.residual_mult)
        blocks.append(block)
        names[f'l{index}.norm1'] = (block.mixer_norm, 'weight')
        for suffix, local in _MIXER_TENSORS[layer['type']].items():
            names[f'l{index}.mix.{suffix}'] = (mixer, local)
        if ffn is not None:
            names[f'l{index}.norm2'] = (block.ffn_norm, 'weight')
            for suffix, local in _FFN_TENSORS.items():
                names[f'l{index}.mlp.{suffix}'] = (ffn, local)
    final_norm, head = LayerNorm(width, eps), LMHead(config.vocab, width)
    names['final.norm'] = (final_norm, 'weight')
    names['head'] = (head, 'weight')
    # a looped layer appears once per run; every run owns a cache (or state) of its mixer's need
    schedule = [ScheduleEntry(index) for index in config.layer_order()]
    return CausalLM(config=config, embedding=embedding, blocks=blocks, schedule=schedule, final_norm=final_norm, head=head,
                    names=names, dtype=dtype, device=device, residual_scale=config.residual_mult)


register_architecture('Fubapel', model_type='fubapel', config_class=FubapelConfig, build=build_fubapel, replace=True)
