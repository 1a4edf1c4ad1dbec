"""Typed configuration of the Fubapel design, read from its own config.json keys.

    architecture   'Fubapel'
    vocab, width   sizes of the embedding
    layers         list; each entry: 'type' (the mixer: 'latent_attention' | 'mlstm' | 'retention'), 'mixer' (its sizes and
                   constants) and 'mlp' (null, or {'kind': 'dense', 'ff', 'limit'})
    loop           {'start', 'stop', 'times'}: layers start .. stop - 1 run 'times' times in a row with the same weights
                   (every run with a cache of its own), then the rest follow; absent: every layer once
    norm           {'eps'}
    residual_mult  what every sub-layer's output is multiplied by as it is added to the stream

Every size and constant comes from here; a key the design does not know is refused, so that a model this engine
would run differently does not load silently.
"""
import copy
from dataclasses import dataclass

from .base import ConfigError, read_config_json, check_positive_int, check_positive_finite

_MIXER_KEYS = {
    'latent_attention': {'heads', 'dim', 'rot_dim', 'vdim', 'kv_rank', 'q_rank', 'rot', 'scale'},
    'mlstm': {'heads', 'dim', 'vdim', 'gate_cap'},
    'retention': {'heads', 'dim', 'vdim', 'decay', 'rot'},
}
_TOP_KEYS = {'architecture', 'architectures', 'model_type', 'vocab', 'width', 'layers', 'loop', 'norm', 'residual_mult'}


def _check_rot(where, rot, most):
    if not isinstance(rot, dict) or set(rot) != {'base', 'dims'}:
        raise ConfigError(f"{where}.rot must be {{'base', 'dims'}}")
    check_positive_finite(f'{where}.rot.base', rot['base'])
    check_positive_int(f'{where}.rot.dims', rot['dims'])
    if rot['dims'] % 2 or rot['dims'] > most:
        raise ConfigError(f'{where}.rot.dims must be even and at most {most}')


def _check_layer(index, layer):
    where = f'layers[{index}]'
    if not isinstance(layer, dict) or set(layer) != {'type', 'mixer', 'mlp'}:
        raise ConfigError(f"{where} must have exactly 'type', 'mixer' and 'mlp'")
    kind, mixer, mlp = layer['type'], layer['mixer'], layer['mlp']
    if kind not in _MIXER_KEYS:
        raise ConfigError(f'{where}.type {kind!r} is not one of {sorted(_MIXER_KEYS)}')
    if not isinstance(mixer, dict) or set(mixer) != _MIXER_KEYS[kind]:
        raise ConfigError(f'{where}.mixer must have exactly the keys {sorted(_MIXER_KEYS[kind])}')
    for name in ('heads', 'dim', 'vdim'):
        check_positive_int(f'{where}.mixer.{name}', mixer[name])
    if kind == 'latent_attention':
        for name in ('rot_dim', 'kv_rank', 'q_rank'):
            check_positive_int(f'{where}.mixer.{name}', mixer[name])
        check_positive_finite(f'{where}.mixer.scale', mixer['scale'])
        _check_rot(f'{where}.mixer', mixer['rot'], mixer['rot_dim'])
        if mixer['rot']['dims'] != mixer['rot_dim']:
            raise ConfigError(f'{where}.mixer: the rotation covers the whole rotated part (rot.dims == rot_dim)')
    elif kind == 'mlstm':
        check_positive_finite(f'{where}.mixer.gate_cap', mixer['gate_cap'])
    else:
        decay = mixer['decay']
        if not isinstance(decay, list) or len(decay) != mixer['heads']:
            raise ConfigError(f'{where}.mixer.decay must list one number per head')
        for value in decay:
            check_positive_finite(f'{where}.mixer.decay', value)
        _check_rot(f'{where}.mixer', mixer['rot'], mixer['dim'])
    if mlp is not None:
        if not isinstance(mlp, dict) or set(mlp) != {'kind', 'ff', 'limit'} or mlp['kind'] != 'dense':
            raise ConfigError(f"{where}.mlp must be null or {{'kind': 'dense', 'ff', 'limit'}}")
        check_positive_int(f'{where}.mlp.ff', mlp['ff'])
        check_positive_finite(f'{where}.mlp.limit', mlp['limit'])


@dataclass(frozen=True)
class FubapelConfig:
    vocab: int
    width: int
    layers: tuple                 # of dicts as in config.json, checked
    loop_start: int
    loop_stop: int
    loop_times: int
    norm_eps: float
    residual_mult: float

    architecture = 'Fubapel'
    model_type = 'fubapel'

    def __post_init__(self):
        check_positive_int('vocab', self.vocab)
        check_positive_int('width', self.width)
        if not self.layers:
            raise ConfigError('layers must not be empty')
        for index, layer in enumerate(self.layers):
            _check_layer(index, layer)
        for name in ('loop_start', 'loop_stop'):
            if type(getattr(self, name)) is not int or getattr(self, name) < 0:
                raise ConfigError(f'loop.{name[5:]} must be a non-negative integer')
        check_positive_int('loop.times', self.loop_times)
        if not self.loop_start <= self.loop_stop <= len(self.layers):
            raise ConfigError('loop: 0 <= start <= stop <= number of layers')
        check_positive_finite('norm.eps', self.norm_eps)
        check_positive_finite('residual_mult', self.residual_mult)

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def eos_ids(self):
        return frozenset()

    def layer_order(self):
        """Indices of the layers in the order they run."""
        span = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + span * self.loop_times + list(range(self.loop_stop, len(self.layers)))

    @classmethod
    def from_dict(cls, data):
        if data.get('architecture', (data.get('architectures') or [None])[0]) != cls.architecture:
            raise ConfigError(f"architecture must be {cls.architecture!r}")
        unknown = sorted(set(data) - _TOP_KEYS)
        if unknown:
            raise ConfigError(f'config.json has keys this design does not know: {unknown}')
        missing = [name for name in ('vocab', 'width', 'layers', 'norm', 'residual_mult') if name not in data]
        if missing:
            raise ConfigError(f'config.json lacks required keys: {missing}')
        if not isinstance(data['layers'], list):
            raise ConfigError('layers must be a list')
        if not isinstance(data['norm'], dict) or set(data['norm']) != {'eps'}:
            raise ConfigError("norm must be {'eps'}")
        loop = data.get('loop')
        if loop is None:
            loop = dict(start=0, stop=0, times=1)
        if not isinstance(loop, dict) or set(loop) != {'start', 'stop', 'times'}:
            raise ConfigError("loop must be {'start', 'stop', 'times'}")
        return cls(vocab=data['vocab'], width=data['width'], layers=tuple(copy.deepcopy(data['layers'])),
                   loop_start=loop['start'], loop_stop=loop['stop'], loop_times=loop['times'],
                   norm_eps=data['norm']['eps'], residual_mult=data['residual_mult'])

    @classmethod
    def read(cls, directory):
        return cls.from_dict(read_config_json(directory))

    def to_dict(self):
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                    layers=copy.deepcopy(list(self.layers)),
                    loop=dict(start=self.loop_start, stop=self.loop_stop, times=self.loop_times),
                    norm=dict(eps=self.norm_eps), residual_mult=self.residual_mult)
