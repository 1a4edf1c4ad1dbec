"""Typed configuration of the Gerivik design, read from its own config.json keys.

    architecture   'Gerivik'
    vocab, width   sizes of the embedding
    embedding      {'scale'}: what an embedded token is multiplied by
    layers         list; each entry: 'type' (the mixer: 'attention' | 'gla'), 'mixer' (its sizes and constants), 'mlp'
                   (null, or {'kind': 'moe', 'expert': {'ff', 'limit'}, 'router': {'experts', 'identity', 'top',
                   'groups': {'count', 'keep'}}}) and optionally 'weights_of': j, the index of another layer with
                   tensors of its own whose tensors this layer uses (with a cache or state of its own); the rest of
                   such an entry equals layer j's
    norm           {'eps'}

Every size and constant comes from here (the inner size of the gla decay's low-rank product comes from the tensors);
a key the design does not know is refused, so that a model this engine would run differently does not load silently.
"""
import copy
from dataclasses import dataclass

from .base import ConfigError, check_positive_int, check_positive_finite, read_config_json

_MIXER_KEYS = {
    'attention': {'heads', 'kv_heads', 'dim', 'vdim', 'rot', 'scale', 'softcap'},
    'gla': {'heads', 'dim', 'vdim', 'tau'},
}
_TOP_KEYS = {'architecture', 'architectures', 'model_type', 'vocab', 'width', 'embedding', 'layers', 'norm'}


def _exact(where, value, keys):
    if not isinstance(value, dict) or set(value) != set(keys):
        raise ConfigError(f'{where} must have exactly the keys {sorted(keys)}')


def _check_layer(index, layer, layers):
    where = f'layers[{index}]'
    if not isinstance(layer, dict) or not {'type', 'mixer', 'mlp'} <= set(layer) <= {'type', 'mixer', 'mlp', 'weights_of'}:
        raise ConfigError(f"{where} must have 'type', 'mixer', 'mlp' and at most 'weights_of' besides")
    kind, mixer, mlp = layer['type'], layer['mixer'], layer['mlp']
    if kind not in _MIXER_KEYS:
        raise ConfigError(f'{where}.type {kind!r} is not one of {sorted(_MIXER_KEYS)}')
    _exact(f'{where}.mixer', mixer, _MIXER_KEYS[kind])
    for name in ('heads', 'dim', 'vdim'):
        check_positive_int(f'{where}.mixer.{name}', mixer[name])
    if kind == 'attention':
        check_positive_int(f'{where}.mixer.kv_heads', mixer['kv_heads'])
        if mixer['heads'] % mixer['kv_heads']:
            raise ConfigError(f'{where}.mixer: heads must be a multiple of kv_heads')
        check_positive_finite(f'{where}.mixer.scale', mixer['scale'])
        check_positive_finite(f'{where}.mixer.softcap', mixer['softcap'])
        _exact(f'{where}.mixer.rot', mixer['rot'], {'base', 'dims'})
        check_positive_finite(f'{where}.mixer.rot.base', mixer['rot']['base'])
        check_positive_int(f'{where}.mixer.rot.dims', mixer['rot']['dims'])
        if mixer['rot']['dims'] % 2 or mixer['rot']['dims'] > mixer['dim']:
            raise ConfigError(f'{where}.mixer.rot.dims must be even and at most dim')
    else:
        check_positive_finite(f'{where}.mixer.tau', mixer['tau'])
    if mlp is not None:
        _exact(f'{where}.mlp', mlp, {'kind', 'expert', 'router'})
        if mlp['kind'] != 'moe':
            raise ConfigError(f"{where}.mlp.kind must be 'moe'")
        _exact(f'{where}.mlp.expert', mlp['expert'], {'ff', 'limit'})
        check_positive_int(f'{where}.mlp.expert.ff', mlp['expert']['ff'])
        check_positive_finite(f'{where}.mlp.expert.limit', mlp['expert']['limit'])
        router = mlp['router']
        _exact(f'{where}.mlp.router', router, {'experts', 'identity', 'top', 'groups'})
        check_positive_int(f'{where}.mlp.router.experts', router['experts'])
        check_positive_int(f'{where}.mlp.router.top', router['top'])
        if type(router['identity']) is not int or router['identity'] < 0:
            raise ConfigError(f'{where}.mlp.router.identity must be a non-negative integer')
        _exact(f'{where}.mlp.router.groups', router['groups'], {'count', 'keep'})
        count, keep = router['groups']['count'], router['groups']['keep']
        check_positive_int(f'{where}.mlp.router.groups.count', count)
        check_positive_int(f'{where}.mlp.router.groups.keep', keep)
        outputs = router['experts'] + router['identity']
        if outputs % count or keep > count or router['top'] > keep * (outputs // count):
            raise ConfigError(f'{where}.mlp.router: {outputs} outputs must split into {count} equal groups of which '
                              f'{keep} can hold {router["top"]} choices')
    if 'weights_of' in layer:
        source = layer['weights_of']
        if type(source) is not int or not 0 <= source < len(layers) or source == index or \
                not isinstance(layers[source], dict) or 'weights_of' in layers[source]:
            raise ConfigError(f'{where}.weights_of must name another layer that has tensors of its own')
        if {k: v for k, v in layer.items() if k != 'weights_of'} != layers[source]:
            raise ConfigError(f'{where}: a layer that uses the tensors of layer {source} must equal it otherwise')


@dataclass(frozen=True)
class GerivikConfig:
    vocab: int
    width: int
    embedding_scale: float
    layers: tuple                 # of dicts as in config.json, checked
    norm_eps: float

    architecture = 'Gerivik'
    model_type = 'gerivik'

    def __post_init__(self):
        check_positive_int('vocab', self.vocab)
        check_positive_int('width', self.width)
        check_positive_finite('embedding.scale', self.embedding_scale)
        if not self.layers:
            raise ConfigError('layers must not be empty')
        for index, layer in enumerate(self.layers):
            _check_layer(index, layer, self.layers)
        check_positive_finite('norm.eps', self.norm_eps)

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def eos_ids(self):
        return frozenset()

    def weights_layer(self, index):
        """The layer whose tensors layer ``index`` uses: itself, or the one it names."""
        return self.layers[index].get('weights_of', index)

    @classmethod
    def from_dict(cls, data):
        if data.get('architecture', (data.get('architectures') or [None])[0]) != cls.architecture:
            raise ConfigError(f"architecture must be {cls.architecture!r}")
        unknown = sorted(set(data) - _TOP_KEYS)
        if unknown:
            raise ConfigError(f'config.json has keys this design does not know: {unknown}')
        missing = [name for name in ('vocab', 'width', 'embedding', 'layers', 'norm') if name not in data]
        if missing:
            raise ConfigError(f'config.json lacks required keys: {missing}')
        if not isinstance(data['layers'], list):
            raise ConfigError('layers must be a list')
        _exact('norm', data['norm'], {'eps'})
        _exact('embedding', data['embedding'], {'scale'})
        return cls(vocab=data['vocab'], width=data['width'], embedding_scale=data['embedding']['scale'],
                   layers=tuple(copy.deepcopy(data['layers'])), norm_eps=data['norm']['eps'])

    @classmethod
    def read(cls, directory):
        return cls.from_dict(read_config_json(directory))

    def to_dict(self):
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                    embedding=dict(scale=self.embedding_scale), layers=copy.deepcopy(list(self.layers)),
                    norm=dict(eps=self.norm_eps))
