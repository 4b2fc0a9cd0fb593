"""Dogozen assembled from parts.

Token embedding; layers of two kinds, chosen layer by layer by the configuration: 'attention' (grouped-query attention
without a rotation, queries and keys with biases and brought to unit root mean square per head, a query temperature
that grows with the logarithm of the position, an output gate from the mixer's own input; a layer may read an earlier
layer's cached keys and values instead of making its own) and 'parallel' (two mixers on the same input whose results
are added with a factor each: windowed attention with partly rotated queries and keys, slowed long waves and a sink
per head; and a selective state-space scan behind a short convolution).  Behind a mixer: a dense gated feed-forward, a
routed one (sigmoid scores, groups scored by their two best, renormalised weights times a constant, a shared expert) or
nothing.  An RMS norm whose weight is stored around zero stands before and after every sub-layer; the final norm is of
that kind too, the head is the embedding table, and the logits pass a soft cap.
"""
import torch

from ..config.dogozen import DogozenConfig
from ..parts import (RMSNorm, RotaryFrequencies, Attention, SelectiveScan, ParallelMixers, GatedMLP, RoutedExperts,
                     SandwichBlock, Embedding, LMHead, CausalLM, ScheduleEntry)
from ..registry import register_architecture

RENORMALIZE_EPS = 1e-20      # what the sum of the chosen scores is increased by before it divides them: fixed by the design


def _attention(width, m, eps, dtype, device):
    temperature = m.get('q_temp')
    return Attention(width=width, heads=m['heads'], kv_heads=m['kv_heads'], head_dim=m['dim'], value_dim=m['vdim'],
                     bias=True, out_bias=False, qk_norm_eps=eps, qk_norm_weights=False, scale=m['scale'], position=None,
                     q_temperature=(temperature['coef'], temperature['every']) if temperature is not None else None,
                     gate=True, own_kv=m.get('kv_from') is None, dtype=dtype)


def _parallel(width, m, eps, dtype, device):
    a, r = m['left'], m['right']
    rot = a.get('rot')
    position = None
    if rot is not None:
        s = rot.get('scaling')
        position = RotaryFrequencies(rot['dims'], rot['base'], device=device,
                                     scaling=(s['factor'], s['low'], s['high'], s['original']) if s is not None else None)
    left = Attention(width=width, heads=a['heads'], kv_heads=a['kv_heads'], head_dim=a['dim'], value_dim=a['vdim'],
                     bias=False, qk_norm_eps=None, scale=a['scale'], position=position,
                     window=a['mask']['size'] if a.get('mask') is not None else None, sink=True, dtype=dtype)
    right = SelectiveScan(width=width, inner=r['inner'], state=r['state'], taps=r['conv'], dt_rank=r['dt_rank'], dtype=dtype)
    return ParallelMixers(left=left, right=right, left_scale=m['left_scale'], right_scale=m['right_scale'])


def _dense(width, f, dtype):
    return GatedMLP(width=width, intermediate=f['ff'], activation='silu', dtype=dtype)


def _moe(width, f, dtype):
    r = f['router']
    groups = r.get('groups') or {'count': 1, 'keep': 1}
    shared = GatedMLP(width=width, intermediate=f['shared']['ff'], activation='silu', dtype=dtype) \
        if f.get('shared') is not None else None
    return RoutedExperts(width=width, experts=r['experts'], top=r['top'], groups=groups['count'], keep=groups['keep'],
                         intermediate=f['expert']['ff'], activation='silu', score='sigmoid', group_score='top2',
                         renormalize=True, renormalize_eps=RENORMALIZE_EPS, weight_scale=r['scale'], shared=shared,
                         dtype=dtype)


MIXERS = {'attention': _attention, 'parallel': _parallel}
FEED_FORWARDS = {'dense': _dense, 'moe': _moe}

# checkpoint suffix -> the part's own tensor name
_ATTENTION_TENSORS = {'q': 'q_proj.weight', 'q.b': 'q_proj.bias', 'k': 'k_proj.weight', 'k.b': 'k_proj.bias',
                      'v': 'v_proj.weight', 'v.b': 'v_proj.bias', 'g': 'g_proj.weight', 'o': 'o_proj.weight'}
_PARALLEL_TENSORS = {'left.q': 'left.q_proj.weight', 'left.k': 'left.k_proj.weight', 'left.v': 'left.v_proj.weight',
                     'left.sink': 'left.sinks', 'left.o': 'left.o_proj.weight',
                     'right.in': 'right.in_proj.weight', 'right.conv': 'right.conv.weight', 'right.conv.b': 'right.conv.bias',
                     'right.x': 'right.x_proj.weight', 'right.dt': 'right.dt_proj.weight', 'right.dt.b': 'right.dt_proj.bias',
                     'right.A_log': 'right.A_log', 'right.D': 'right.D', 'right.o': 'right.o_proj.weight'}
_MLP_TENSORS = {'gate': 'gate_proj.weight', 'up': 'up_proj.weight', 'down': 'down_proj.weight'}


def build_dogozen(config, *, dtype=torch.bfloat16, device='cuda'):
    width, eps = config.width, config.norm_eps
    embedding = Embedding(config.vocab, width)
    blocks, names = [], {'embed': (embedding, 'weight')}
    norm = lambda: RMSNorm(width, eps, offset=1.0)
    for index, layer in enumerate(config.layers):
        mixer = MIXERS[layer['type']](width, layer['mixer'], eps, dtype, device)
        ffn = FEED_FORWARDS[layer['mlp']['kind']](width, layer['mlp'], dtype) if layer['mlp'] is not None else None
        block = SandwichBlock(mixer_norm=norm(), mixer=mixer, mixer_post_norm=norm(),
                              ffn_norm=norm() if ffn is not None else None, ffn=ffn,
                              ffn_post_norm=norm() if ffn is not None else None, dtype=dtype)
        blocks.append(block)
        names[f'l{index}.norm1'] = (block.mixer_norm, 'weight')
        names[f'l{index}.norm1b'] = (block.mixer_post_norm, 'weight')
        declared = mixer.param_specs()
        table = _ATTENTION_TENSORS if layer['type'] == 'attention' else _PARALLEL_TENSORS
        for suffix, local in table.items():
            if local in declared:                       # (a layer that reads another's keys and values has none)
                names[f'l{index}.mix.{suffix}'] = (mixer, local)
        if ffn is None:
            continue
        names[f'l{index}.norm2'] = (block.ffn_norm, 'weight')
        names[f'l{index}.norm2b'] = (block.ffn_post_norm, 'weight')
        if layer['mlp']['kind'] == 'dense':
            for suffix, local in _MLP_TENSORS.items():
                names[f'l{index}.mlp.{suffix}'] = (ffn, local)
            continue
        names[f'l{index}.mlp.router'] = (ffn, 'router.weight')
        for e in range(ffn.experts):
            for suffix, local in _MLP_TENSORS.items():
                names[f'l{index}.mlp.e{e}.{suffix}'] = (ffn, f'experts.{e}.{local}')
        if ffn.shared is not None:
            for suffix, local in _MLP_TENSORS.items():
                names[f'l{index}.mlp.shared.{suffix}'] = (ffn, f'shared.{local}')
    final_norm = RMSNorm(width, eps, offset=1.0)
    head = LMHead(config.vocab, width, tied_to=embedding, softcap=config.logit_softcap)
    names['final.norm'] = (final_norm, 'weight')
    # a layer with kv_from reads the cache that the named layer's run owns (schedule positions are layer indices)
    schedule = [ScheduleEntry(index, cache_of=layer['mixer'].get('kv_from') if layer['type'] == 'attention' else None)
                for index, layer in enumerate(config.layers)]
    return CausalLM(config=config, embedding=embedding, blocks=blocks, schedule=schedule, final_norm=final_norm, head=head,
                    names=names, dtype=dtype, device=device)


register_architecture('Dogozen', model_type='dogozen', config_class=DogozenConfig, build=build_dogozen, replace=True)
