"""Typed configuration of the Zinesun design, read from its own config.json keys.

    architecture   'Zinesun'
    vocab, width   sizes of the embedding
    embedding      {'scale'}: what an embedded token is multiplied by
    canon          {'taps'}: the taps of the short convolution in front of every mixer
    layers         list; each entry: 'type' (the mixer: 'latent_attention'), 'mixer' (its sizes and constants:
                   'heads', 'dim', 'rot_dim', 'vdim', 'kv_rank', 'q_rank', 'scale', 'rot': {'base', 'dims'},
                   'mask': {'size'}) and 'mlp': null, {'kind': 'dense', 'ff'} or {'kind': 'moe', 'expert': {'ff'},
                   'router': {'experts', 'top'}}
    norm           {'eps'}

Every size and constant comes from here; a key the design does not know is refused, so that a model this engine
would run differently does not load silently.
"""
import copy
from dataclasses import dataclass

from .base import ConfigError, check_positive_int, check_positive_finite, read_config_json

_MIXER_KEYS = {
    'latent_attention': {'heads', 'dim', 'rot_dim', 'vdim', 'kv_rank', 'q_rank', 'scale', 'rot', 'mask'},
}
_TOP_KEYS = {'architecture', 'architectures', 'model_type', 'vocab', 'width', 'embedding', 'canon', 'layers', 'norm'}


def _exact(where, value, keys):
    if not isinstance(value, dict) or set(value) != set(keys):
        raise ConfigError(f'{where} must have exactly the keys {sorted(keys)}')


def _check_layer(index, layer):
    where = f'layers[{index}]'
    _exact(where, layer, {'type', 'mixer', 'mlp'})
    kind, mixer, mlp = layer['type'], layer['mixer'], layer['mlp']
    if kind not in _MIXER_KEYS:
        raise ConfigError(f'{where}.type {kind!r} is not one of {sorted(_MIXER_KEYS)}')
    _exact(f'{where}.mixer', mixer, _MIXER_KEYS[kind])
    for name in ('heads', 'dim', 'rot_dim', 'vdim', 'kv_rank', 'q_rank'):
        check_positive_int(f'{where}.mixer.{name}', mixer[name])
    check_positive_finite(f'{where}.mixer.scale', mixer['scale'])
    _exact(f'{where}.mixer.rot', mixer['rot'], {'base', 'dims'})
    check_positive_finite(f'{where}.mixer.rot.base', mixer['rot']['base'])
    check_positive_int(f'{where}.mixer.rot.dims', mixer['rot']['dims'])
    if mixer['rot_dim'] % 2 or mixer['rot']['dims'] != mixer['rot_dim']:
        raise ConfigError(f'{where}.mixer: the rotation covers the whole rotated part (rot.dims == rot_dim, even)')
    _exact(f'{where}.mixer.mask', mixer['mask'], {'size'})
    check_positive_int(f'{where}.mixer.mask.size', mixer['mask']['size'])
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get('kind') not in ('dense', 'moe'):
        raise ConfigError(f"{where}.mlp must be null or have 'kind': 'dense' or 'moe'")
    if mlp['kind'] == 'dense':
        _exact(f'{where}.mlp', mlp, {'kind', 'ff'})
        check_positive_int(f'{where}.mlp.ff', mlp['ff'])
    else:
        _exact(f'{where}.mlp', mlp, {'kind', 'expert', 'router'})
        _exact(f'{where}.mlp.expert', mlp['expert'], {'ff'})
        check_positive_int(f'{where}.mlp.expert.ff', mlp['expert']['ff'])
        _exact(f'{where}.mlp.router', mlp['router'], {'experts', 'top'})
        check_positive_int(f'{where}.mlp.router.experts', mlp['router']['experts'])
        check_positive_int(f'{where}.mlp.router.top', mlp['router']['top'])
        if mlp['router']['top'] > mlp['router']['experts']:
            raise ConfigError(f'{where}.mlp.router: top must not exceed experts')


@dataclass(frozen=True)
class ZinesunConfig:
    vocab: int
    width: int
    embedding_scale: float
    taps: int
    layers: tuple                 # of dicts as in config.json, checked
    norm_eps: float

    architecture = 'Zinesun'
    model_type = 'zinesun'

    def __post_init__(self):
        check_positive_int('vocab', self.vocab)
        check_positive_int('width', self.width)
        check_positive_finite('embedding.scale', self.embedding_scale)
        check_positive_int('canon.taps', self.taps)
        if not self.layers:
            raise ConfigError('layers must not be empty')
        for index, layer in enumerate(self.layers):
            _check_layer(index, layer)
        check_positive_finite('norm.eps', self.norm_eps)

    @property
    def vocab_size(self):
        return self.vocab

    @property
    def eos_ids(self):
        return frozenset()

    @classmethod
    def from_dict(cls, data):
        if data.get('architecture', (data.get('architectures') or [None])[0]) != cls.architecture:
            raise ConfigError(f"architecture must be {cls.architecture!r}")
        unknown = sorted(set(data) - _TOP_KEYS)
        if unknown:
            raise ConfigError(f'config.json has keys this design does not know: {unknown}')
        missing = [name for name in ('vocab', 'width', 'embedding', 'canon', 'layers', 'norm') if name not in data]
        if missing:
            raise ConfigError(f'config.json lacks required keys: {missing}')
        if not isinstance(data['layers'], list):
            raise ConfigError('layers must be a list')
        _exact('norm', data['norm'], {'eps'})
        _exact('embedding', data['embedding'], {'scale'})
        _exact('canon', data['canon'], {'taps'})
        return cls(vocab=data['vocab'], width=data['width'], embedding_scale=data['embedding']['scale'],
                   taps=data['canon']['taps'], layers=tuple(copy.deepcopy(data['layers'])), norm_eps=data['norm']['eps'])

    @classmethod
    def read(cls, directory):
        return cls.from_dict(read_config_json(directory))

    def to_dict(self):
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                    embedding=dict(scale=self.embedding_scale), canon=dict(taps=self.taps),
                    layers=copy.deepcopy(list(self.layers)), norm=dict(eps=self.norm_eps))
