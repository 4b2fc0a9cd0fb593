"""Zinesun assembled from parts.

Token embedding times a scale; every layer is attention over a cached latent (queries through a latent of their own,
a rotated key part shared by the heads with neighbouring elements paired, a sliding window, a sigmoid gate per head
on the heads' results) followed by a dense feed-forward with the xielu activation, a routed feed-forward (silu-gated
experts, a router with a bias whose weights are the softmax over the chosen logits) or nothing.  The sub-layers read
the residual stream itself, the mixer through a short causal convolution over time; a layer norm with weight and bias
stands on every sub-layer's output, which is scaled per channel before it is added; what goes on from a layer is a
stored weighted average of the embedding's output and all layers' results so far.  Final layer norm with bias; the
head is the embedding table itself (without the scale).
"""
import torch

from ..config.zinesun import ZinesunConfig
from ..parts import (LayerNorm, RotaryFrequencies, LatentAttention, PlainMLP, RoutedExperts, ShortConvolution,
                     PostNormBlock, Embedding, LMHead, CausalLM, ScheduleEntry)
from ..registry import register_architecture


def _latent_attention(width, m, eps, dtype, device):
    return LatentAttention(width=width, heads=m['heads'], dim=m['dim'], rot_dim=m['rot_dim'], vdim=m['vdim'],
                           kv_rank=m['kv_rank'], q_rank=m['q_rank'], scale=m['scale'], eps=eps, sink=False,
                           window=m['mask']['size'], gate=True, pairing='neighbours',
                           position=RotaryFrequencies(m['rot']['dims'], m['rot']['base'], device=device), dtype=dtype)


def _dense(width, f, dtype):
    return PlainMLP(width=width, intermediate=f['ff'], activation='xielu', dtype=dtype)


def _moe(width, f, dtype):
    return RoutedExperts(width=width, experts=f['router']['experts'], top=f['router']['top'],
                         intermediate=f['expert']['ff'], activation='silu', bias=True, renormalize=True, dtype=dtype)


MIXERS = {'latent_attention': _latent_attention}
FEED_FORWARDS = {'dense': _dense, 'moe': _moe}

# checkpoint suffix -> the part's own tensor name
_MIXER_TENSORS = {
    'latent_attention': {'dq': 'q_down.weight', 'dq.norm': 'q_norm.weight', 'uq': 'q_up.weight', 'dkv': 'kv_down.weight',
                         'dkv.norm': 'kv_norm.weight', 'uk': 'k_up.weight', 'uv': 'v_up.weight', 'g': 'g_proj.weight',
                         'o': 'o_proj.weight'},
}
_DENSE_TENSORS = {'up': 'up_proj.weight', 'down': 'down_proj.weight', 'act': 'act'}
_EXPERT_TENSORS = {'gate': 'gate_proj.weight', 'up': 'up_proj.weight', 'down': 'down_proj.weight'}


def build_zinesun(config, *, dtype=torch.bfloat16, device='cuda'):
    width, eps, depth_total = config.width, config.norm_eps, len(config.layers) + 1
    embedding = Embedding(config.vocab, width, scale=config.embedding_scale)
    blocks, names = [], {'embed': (embedding, 'weight')}
    for index, layer in enumerate(config.layers):
        mixer = MIXERS[layer['type']](width, layer['mixer'], eps, dtype, device)
        ffn = FEED_FORWARDS[layer['mlp']['kind']](width, layer['mlp'], dtype) if layer['mlp'] is not None else None
        norm = lambda: LayerNorm(width, eps, bias=True)
        block = PostNormBlock(mixer=mixer, mixer_post_norm=norm(), ffn=ffn, ffn_post_norm=norm() if ffn is not None else None,
                              input_conv=ShortConvolution(width, config.taps), layer_scale=True, depth=index + 2,
                              depth_total=depth_total, width=width, dtype=dtype)
        blocks.append(block)
        names[f'l{index}.norm1'] = (block.mixer_post_norm, 'weight')
        names[f'l{index}.norm1.b'] = (block.mixer_post_norm, 'bias')
        names[f'l{index}.ls1'] = (block, 'mixer_scale')
        names[f'l{index}.canon1'] = (block.input_conv, 'weight')
        names[f'l{index}.dwa'] = (block, 'depth_mix')
        for suffix, local in _MIXER_TENSORS[layer['type']].items():
            names[f'l{index}.mix.{suffix}'] = (mixer, local)
        if ffn is None:
            continue
        names[f'l{index}.norm2'] = (block.ffn_post_norm, 'weight')
        names[f'l{index}.norm2.b'] = (block.ffn_post_norm, 'bias')
        names[f'l{index}.ls2'] = (block, 'ffn_scale')
        if layer['mlp']['kind'] == 'dense':
            for suffix, local in _DENSE_TENSORS.items():
                names[f'l{index}.mlp.{suffix}'] = (ffn, local)
        else:
            names[f'l{index}.mlp.router'] = (ffn, 'router.weight')
            names[f'l{index}.mlp.router.b'] = (ffn, 'router.bias')
            for e in range(ffn.experts):
                for suffix, local in _EXPERT_TENSORS.items():
                    names[f'l{index}.mlp.e{e}.{suffix}'] = (ffn, f'experts.{e}.{local}')
    final_norm, head = LayerNorm(width, eps, bias=True), LMHead(config.vocab, width, tied_to=embedding)
    names['final.norm'] = (final_norm, 'weight')
    names['final.norm.b'] = (final_norm, 'bias')
    schedule = [ScheduleEntry(index) for index in range(len(blocks))]
    return CausalLM(config=config, embedding=embedding, blocks=blocks, schedule=schedule, final_norm=final_norm, head=head,
                    names=names, dtype=dtype, device=device)


register_architecture('Zinesun', model_type='zinesun', config_class=ZinesunConfig, build=build_zinesun, replace=True)
