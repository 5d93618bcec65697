"""Llama entry points of the drop-in: `load_usa`, `convert_usa`, `reset_usa`, `set_train_usa_mode`,
`set_eval_usa_mode`, `print_stats`, `USA`, `LlamaAttention_heavy_hitter` - the names, arguments and behaviour of
the reference's hashattention/hashattention_llama.py (:87-226, :229-631, :633-725), written against the installed
`transformers` 5.x attention interface (`past_key_values`, two return values).

    from hashattention.hashattention_llama import load_usa, convert_usa, reset_usa
    usa = load_usa(config, "usa_checkpoint.pt")          # config carries lth_* and *_budget fields
    model = convert_usa(model, config, usa, collect_stats=False, train_usa=False)
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn
from transformers.models.llama.modeling_llama import LlamaAttention, apply_rotary_pos_emb

from ._patched import (DEFAULT_USA_CFG, USA, HeavyHitterMixin, SignSTE, build_usa_modules, convert_modules, install_fast_layers,
                       memory_efficient_softmax, ste_sign, walk)

__all__ = ["USA", "LlamaAttention_heavy_hitter", "load_usa", "convert_usa", "reset_usa", "set_train_usa_mode",
           "set_eval_usa_mode", "print_stats", "SignSTE", "ste_sign", "memory_efficient_softmax", "DEFAULT_USA_CFG"]


class LlamaAttention_heavy_hitter(HeavyHitterMixin, nn.Module):
    """Llama attention whose decode steps (q_len <= 128) attend only to sink | recent | hash-selected tokens."""

    def __init__(self, config, layer_idx: Optional[int] = None):
        nn.Module.__init__(self)
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.scaling = self.head_dim ** -0.5
        self.attention_dropout = config.attention_dropout
        self.is_causal = True
        bias = getattr(config, "attention_bias", False)
        self.q_proj = nn.Linear(config.hidden_size, config.num_attention_heads * self.head_dim, bias=bias)
        self.k_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.v_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.o_proj = nn.Linear(config.num_attention_heads * self.head_dim, config.hidden_size, bias=bias)
        self._init_heavy_hitter(config)

    @staticmethod
    def _apply_rope(q, k, cos, sin):
        return apply_rotary_pos_emb(q, k, cos, sin)

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                past_key_value=None, **kwargs):
        cache = past_key_values if past_key_values is not None else past_key_value
        return self._heavy_hitter_forward(hidden_states, position_embeddings, attention_mask, cache, **kwargs)


def load_usa(config, path):
    """One `USA` per layer from `config.lth_*`, optionally loaded from the state dict at `path`, on the GPU."""
    return build_usa_modules(config, path)


def convert_usa(model, config, usa_modules, collect_stats, train_usa):
    """Replace every `LlamaAttention` of `model` in place by a `LlamaAttention_heavy_hitter` sharing its weights."""
    return install_fast_layers(convert_modules(model, config, usa_modules, collect_stats, train_usa, LlamaAttention,
                                              LlamaAttention_heavy_hitter))


def reset_usa(model):
    return walk(model, LlamaAttention_heavy_hitter, lambda m: m._reset_state())


def set_train_usa_mode(model, loss_func=None, optimizer=None):
    def fn(m):
        m.train_usa = True
        if loss_func is not None:
            m.tr_loss_func = loss_func
        if optimizer is not None:
            m.tr_optimizer = optimizer
    return walk(model, LlamaAttention_heavy_hitter, fn)


def set_eval_usa_mode(model):
    def fn(m):
        m.train_usa = False
    return walk(model, LlamaAttention_heavy_hitter, fn)


def print_stats(model):
    def fn(m):
        if m.layer_idx == 5:
            print(m.layer_idx)
            print(m.overlaps)
    return walk(model, LlamaAttention_heavy_hitter, fn)
