"""Mistral entry points of the drop-in (reference: hashattention/hashattention_mistral.py): the same API as
`hashattention_llama`, with the Mistral specifics of the reference - bias-free projections (:198-201), a hash
MLP that is always three layers deep because its config has no `lth_num_layers` (:77-88, :566-570)."""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn
from transformers.models.mistral.modeling_mistral import MistralAttention, apply_rotary_pos_emb

from ._patched import (DEFAULT_USA_CFG, USA, HeavyHitterMixin, SignSTE, build_usa_modules, convert_modules, install_fast_layers,
                       memory_efficient_softmax, ste_sign, walk)

__all__ = ["USA", "MistralAttention_heavy_hitter", "load_usa", "convert_usa", "reset_usa", "set_train_usa_mode",
           "set_eval_usa_mode", "print_stats", "SignSTE", "ste_sign", "memory_efficient_softmax", "DEFAULT_USA_CFG"]


class MistralAttention_heavy_hitter(HeavyHitterMixin, nn.Module):
    def __init__(self, config, layer_idx: Optional[int] = None):
        nn.Module.__init__(self)
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.scaling = self.head_dim ** -0.5
        self.attention_dropout = config.attention_dropout
        self.is_causal = True
        self.q_proj = nn.Linear(config.hidden_size, config.num_attention_heads * self.head_dim, bias=False)
        self.k_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=False)
        self.v_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=False)
        self.o_proj = nn.Linear(config.num_attention_heads * self.head_dim, config.hidden_size, bias=False)
        self._init_heavy_hitter(config)

    @staticmethod
    def _apply_rope(q, k, cos, sin):
        return apply_rotary_pos_emb(q, k, cos, sin)

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                past_key_value=None, **kwargs):
        cache = past_key_values if past_key_values is not None else past_key_value
        return self._heavy_hitter_forward(hidden_states, position_embeddings, attention_mask, cache, **kwargs)


def load_usa(config, path):
    """As the Llama `load_usa`, except that `config.lth_num_layers` is not read: the reference's Mistral `USA` has the
    three-layer MLP only (hashattention_mistral.py:77-88, :566-570)."""
    return build_usa_modules(config, path, force_num_layers=3)


def convert_usa(model, config, usa_modules, collect_stats, train_usa):
    return install_fast_layers(convert_modules(model, config, usa_modules, collect_stats, train_usa, MistralAttention,
                                              MistralAttention_heavy_hitter))


def reset_usa(model):
    return walk(model, MistralAttention_heavy_hitter, lambda m: m._reset_state())


def set_train_usa_mode(model, loss_func=None, optimizer=None):
    def fn(m):
        m.train_usa = True
        if loss_func is not None:
            m.tr_loss_func = loss_func
        if optimizer is not None:
            m.tr_optimizer = optimizer
    return walk(model, MistralAttention_heavy_hitter, fn)


def set_eval_usa_mode(model):
    def fn(m):
        m.train_usa = False
    return walk(model, MistralAttention_heavy_hitter, fn)


def print_stats(model):
    def fn(m):
        if m.layer_idx == 5:
            print(m.layer_idx)
            print(m.overlaps)
    return walk(model, MistralAttention_heavy_hitter, fn)
