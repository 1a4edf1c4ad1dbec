"""Gerivik assembled from parts.

Token embedding times a scale; layers of two kinds of mixer, chosen layer by layer by the configuration (grouped-query
attention whose queries and keys are partly rotated, brought to unit root mean square after the rotation, and whose
scores are soft-capped; gated linear attention, a matrix memory whose rows decay each by a factor of their own), each
followed by a routed feed-forward (experts chosen within the best groups, identity experts among them) or by nothing;
an RMS norm before and after every sub-layer; a layer may use an earlier layer's tensors with a cache or state of its
own; final RMS norm and an untied head.
"""
import torch

from ..config.gerivik import GerivikConfig
from ..parts import (RMSNorm, RotaryFrequencies, Attention, MatrixMemory, RoutedExperts, SandwichBlock, Embedding, LMHead,
                     CausalLM, ScheduleEntry)
from ..registry import register_architecture

SWISH_SLOPE = 1.702          # the slope inside the experts' gate sigmoid: fixed by the design


def _attention(width, m, eps, dtype, device):
    return Attention(width=width, heads=m['heads'], kv_heads=m['kv_heads'], head_dim=m['dim'], value_dim=m['vdim'],
                     bias=False, qk_norm_eps=eps, qk_norm_weights=False, norm_after_rotation=True, scale=m['scale'],
                     softcap=m['softcap'], position=RotaryFrequencies(m['rot']['dims'], m['rot']['base'], device=device),
                     dtype=dtype)


def _gla(width, m, eps, dtype, device):
    return MatrixMemory(width=width, heads=m['heads'], dim=m['dim'], vdim=m['vdim'], gating='channel', tau=m['tau'],
                        eps=eps, gate='silu', out_norm=True, out_norm_shared=True, q_scale=m['dim'] ** -0.5, dtype=dtype)


def _moe(width, f, dtype):
    r = f['router']
    return RoutedExperts(width=width, experts=r['experts'], identity=r['identity'], top=r['top'],
                         groups=r['groups']['count'], keep=r['groups']['keep'], intermediate=f['expert']['ff'],
                         activation='clamped_swish', limit=f['expert']['limit'], alpha=SWISH_SLOPE, correction=True,
                         renormalize=False, dtype=dtype)


MIXERS = {'attention': _attention, 'gla': _gla}
FEED_FORWARDS = {'moe': _moe}

# checkpoint suffix -> the part's own tensor name
_MIXER_TENSORS = {
    'attention': {'q': 'q_proj.weight', 'k': 'k_proj.weight', 'v': 'v_proj.weight', 'o': 'o_proj.weight'},
    'gla': {'q': 'q_proj.weight', 'k': 'k_proj.weight', 'v': 'v_proj.weight', 'g': 'g_proj.weight', 'o': 'o_proj.weight',
            'norm': 'out_norm.weight', 'a1': 'decay_down.weight', 'a2': 'decay_up.weight', 'a2.b': 'decay_up.bias'},
}
_EXPERT_TENSORS = {'gate': 'gate_proj.weight', 'up': 'up_proj.weight', 'down': 'down_proj.weight'}


def build_gerivik(config, *, dtype=torch.bfloat16, device='cuda'):
    width, eps = config.width, config.norm_eps
    embedding = Embedding(config.vocab, width, scale=config.embedding_scale)
    blocks, names, block_of = [], {'embed': (embedding, 'weight')}, {}
    for index, layer in enumerate(config.layers):
        if 'weights_of' in layer:                       # no tensors of its own: one more run of that layer's block
            continue
        mixer = MIXERS[layer['type']](width, layer['mixer'], eps, dtype, device)
        ffn = FEED_FORWARDS[layer['mlp']['kind']](width, layer['mlp'], dtype) if layer['mlp'] is not None else None
        norm = lambda: RMSNorm(width, eps)
        block = SandwichBlock(mixer_norm=norm(), mixer=mixer, mixer_post_norm=norm(),
                              ffn_norm=norm() if ffn is not None else None, ffn=ffn,
                              ffn_post_norm=norm() if ffn is not None else None, dtype=dtype)
        block_of[index] = len(blocks)
        blocks.append(block)
        names[f'l{index}.norm1'] = (block.mixer_norm, 'weight')
        names[f'l{index}.norm1b'] = (block.mixer_post_norm, 'weight')
        for suffix, local in _MIXER_TENSORS[layer['type']].items():
            names[f'l{index}.mix.{suffix}'] = (mixer, local)
        if ffn is not None:
            names[f'l{index}.norm2'] = (block.ffn_norm, 'weight')
            names[f'l{index}.norm2b'] = (block.ffn_post_norm, 'weight')
            names[f'l{index}.mlp.router'] = (ffn, 'router.weight')
            names[f'l{index}.mlp.correction'] = (ffn, 'router.correction')
            for e in range(ffn.experts):
                for suffix, local in _EXPERT_TENSORS.items():
                    names[f'l{index}.mlp.e{e}.{suffix}'] = (ffn, f'experts.{e}.{local}')
    final_norm, head = RMSNorm(width, eps), LMHead(config.vocab, width)
    names['final.norm'] = (final_norm, 'weight')
    names['head'] = (head, 'weight')
    # a layer that uses another's tensors is a second run of that block; every run owns a cache (or state) of its own
    schedule = [ScheduleEntry(block_of[config.weights_layer(index)]) for index in range(len(config.layers))]
    return CausalLM(config=config, embedding=embedding, blocks=blocks, schedule=schedule, final_norm=final_norm, head=head,
                    names=names, dtype=dtype, device=device)


register_architecture('Gerivik', model_type='gerivik', config_class=GerivikConfig, build=build_gerivik, replace=True)
