"""Typed configuration of the Dogozen design, read from its own config.json keys.

    architecture   'Dogozen'
    vocab, width   sizes of the embedding (the head is the embedding table)
    layers         list; each entry: 'type' ('attention' | 'parallel'), 'mixer' (its sizes and constants) and 'mlp'
                   (null, {'kind': 'dense', 'ff'}, or {'kind': 'moe', 'expert': {'ff'}, 'router': {'experts', 'top',
                   'scale', 'groups': {'count', 'keep'}}, 'shared': {'ff'}})
      attention    {'heads', 'kv_heads', 'dim', 'vdim', 'scale'}, optionally 'q_temp': {'coef', 'every'} and
                   'kv_from': j (the layer reads layer j's cached keys and values and has no key and value tensors)
      parallel     {'left': {'heads', 'kv_heads', 'dim', 'vdim', 'scale', 'rot': {'base', 'dims', 'scaling': {'factor',
                   'low', 'high', 'original'}}, 'mask': {'size'}}, 'right': {'inner', 'state', 'conv', 'dt_rank'},
                   'left_scale', 'right_scale'}
    norm           {'eps'}
    logit_softcap  c: logits become c * tanh(logits / c); absent or null: no cap

Every size and constant comes from here; a key the design does not know is refused, so that a model this engine would
run differently does not load silently.
"""
import copy
import math
from dataclasses import dataclass

from .base import ConfigError, check_positive_int, check_positive_finite, read_config_json

_TOP_KEYS = {'architecture', 'architectures', 'model_type', 'vocab', 'width', 'layers', 'norm', 'logit_softcap'}


def _keys(where, value, required, optional=()):
    if not isinstance(value, dict) or not set(required) <= set(value) <= set(required) | set(optional):
        raise ConfigError(f'{where} must have the keys {sorted(required)}' +
                          (f' and at most {sorted(optional)} besides' if optional else ''))


def _finite(name, value):
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value):
        raise ConfigError(f'{name} must be a finite number, got {value!r}')


def _check_heads(where, m):
    for name in ('heads', 'kv_heads', 'dim', 'vdim'):
        check_positive_int(f'{where}.{name}', m[name])
    if m['heads'] % m['kv_heads']:
        raise ConfigError(f'{where}: heads must be a multiple of kv_heads')
    check_positive_finite(f'{where}.scale', m['scale'])


def _check_attention(where, m, index, layers):
    _keys(where, m, {'heads', 'kv_heads', 'dim', 'vdim', 'scale'}, {'q_temp', 'kv_from'})
    _check_heads(where, m)
    if m.get('q_temp') is not None:
        _keys(f'{where}.q_temp', m['q_temp'], {'coef', 'every'})
        _finite(f'{where}.q_temp.coef', m['q_temp']['coef'])
        check_positive_int(f'{where}.q_temp.every', m['q_temp']['every'])
    source = m.get('kv_from')
    if source is not None:
        ok = type(source) is int and 0 <= source < index and isinstance(layers[source], dict) and \
            layers[source].get('type') == 'attention' and isinstance(layers[source].get('mixer'), dict) and \
            layers[source]['mixer'].get('kv_from') is None
        if not ok:
            raise ConfigError(f'{where}.kv_from must name an earlier attention layer with keys and values of its own')
        theirs = layers[source]['mixer']
        if any(theirs.get(name) != m[name] for name in ('kv_heads', 'dim', 'vdim')):
            raise ConfigError(f'{where}.kv_from: layer {source} caches keys and values of other sizes')


def _check_parallel(where, m):
    _keys(where, m, {'left', 'right', 'left_scale', 'right_scale'})
    _finite(f'{where}.left_scale', m['left_scale'])
    _finite(f'{where}.right_scale', m['right_scale'])
    left, right = m['left'], m['right']
    _keys(f'{where}.left', left, {'heads', 'kv_heads', 'dim', 'vdim', 'scale'}, {'rot', 'mask'})
    _check_heads(f'{where}.left', left)
    if left.get('rot') is not None:
        rot = left['rot']
        _keys(f'{where}.left.rot', rot, {'base', 'dims'}, {'scaling'})
        check_positive_finite(f'{where}.left.rot.base', rot['base'])
        check_positive_int(f'{where}.left.rot.dims', rot['dims'])
        if rot['dims'] % 2 or rot['dims'] > left['dim']:
            raise ConfigError(f'{where}.left.rot.dims must be even and at most dim')
        if rot.get('scaling') is not None:
            _keys(f'{where}.left.rot.scaling', rot['scaling'], {'factor', 'low', 'high', 'original'})
            for name in ('factor', 'low', 'high', 'original'):
                check_positive_finite(f'{where}.left.rot.scaling.{name}', rot['scaling'][name])
            if not rot['scaling']['high'] > rot['scaling']['low']:
                raise ConfigError(f'{where}.left.rot.scaling: high must exceed low')
    if left.get('mask') is not None:
        _keys(f'{where}.left.mask', left['mask'], {'size'})
        check_positive_int(f'{where}.left.mask.size', left['mask']['size'])
    _keys(f'{where}.right', right, {'inner', 'state', 'conv', 'dt_rank'})
    for name in ('inner', 'state', 'conv', 'dt_rank'):
        check_positive_int(f'{where}.right.{name}', right[name])


def _check_mlp(where, mlp):
    if not isinstance(mlp, dict) or mlp.get('kind') not in ('dense', 'moe'):
        raise ConfigError(f"{where}.kind must be 'dense' or 'moe'")
    if mlp['kind'] == 'dense':
        _keys(where, mlp, {'kind', 'ff'})
        check_positive_int(f'{where}.ff', mlp['ff'])
        return
    _keys(where, mlp, {'kind', 'expert', 'router'}, {'shared'})
    _keys(f'{where}.expert', mlp['expert'], {'ff'})
    check_positive_int(f'{where}.expert.ff', mlp['expert']['ff'])
    router = mlp['router']
    _keys(f'{where}.router', router, {'experts', 'top', 'scale'}, {'groups'})
    check_positive_int(f'{where}.router.experts', router['experts'])
    check_positive_int(f'{where}.router.top', router['top'])
    _finite(f'{where}.router.scale', router['scale'])
    count, keep = 1, 1
    if router.get('groups') is not None:
        _keys(f'{where}.router.groups', router['groups'], {'count', 'keep'})
        count, keep = router['groups']['count'], router['groups']['keep']
        check_positive_int(f'{where}.router.groups.count', count)
        check_positive_int(f'{where}.router.groups.keep', keep)
    if router['experts'] % count or keep > count or router['top'] > keep * (router['experts'] // count):
        raise ConfigError(f'{where}.router: {router["experts"]} experts must split into {count} equal groups of which '
                          f'{keep} can hold {router["top"]} choices')
    if mlp.get('shared') is not None:
        _keys(f'{where}.shared', mlp['shared'], {'ff'})
        check_positive_int(f'{where}.shared.ff', mlp['shared']['ff'])


def _check_layer(index, layer, layers):
    where = f'layers[{index}]'
    _keys(where, layer, {'type', 'mixer', 'mlp'})
    if layer['type'] == 'attention':
        _check_attention(f'{where}.mixer', layer['mixer'], index, layers)
    elif layer['type'] == 'parallel':
        _check_parallel(f'{where}.mixer', layer['mixer'])
    else:
        raise ConfigError(f"{where}.type {layer['type']!r} is not one of ['attention', 'parallel']")
    if layer['mlp'] is not None:
        _check_mlp(f'{where}.mlp', layer['mlp'])


@dataclass(frozen=True)
class DogozenConfig:
    vocab: int
    width: int
    layers: tuple                 # of dicts as in config.json, checked
    norm_eps: float
    logit_softcap: float | None = None

    architecture = 'Dogozen'
    model_type = 'dogozen'

    def __post_init__(self):
        check_positive_int('vocab', self.vocab)
        check_positive_int('width', self.width)
        if not self.layers:
            raise ConfigError('layers must not be empty')
        for index, layer in enumerate(self.layers):
            _check_layer(index, layer, self.layers)
        check_positive_finite('norm.eps', self.norm_eps)
        if self.logit_softcap is not None:
            check_positive_finite('logit_softcap', self.logit_softcap)

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
        missing = [name for name in ('vocab', 'width', 'layers', 'norm') if name not in data]
        if missing:
            raise ConfigError(f'config.json lacks required keys: {missing}')
        if not isinstance(data['layers'], list):
            raise ConfigError('layers must be a list')
        _keys('norm', data['norm'], {'eps'})
        return cls(vocab=data['vocab'], width=data['width'], layers=tuple(copy.deepcopy(data['layers'])),
                   norm_eps=data['norm']['eps'], logit_softcap=data.get('logit_softcap'))

    @classmethod
    def read(cls, directory):
        return cls.from_dict(read_config_json(directory))

    def to_dict(self):
        out = dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                   layers=copy.deepcopy(list(self.layers)), norm=dict(eps=self.norm_eps))
        if self.logit_softcap is not None:
            out['logit_softcap'] = self.logit_softcap
        return out
