"""Seeded synthetic inputs for the sparse-decode path (tests, smoke run and benchmark).

The workloads are the attention-layer shapes the reference benchmarks at
(`efficiency/kernels/torchatt.py:143-165`: H=32, D=128, one decode query per
sequence) with Llama-3.1-8B grouping (32 query heads, 8 KV heads).  Every tensor
is drawn on the CPU from `torch.Generator` so that the same bytes are produced
in any process; `sha256_of` fingerprints them for the golden fixtures.

Draw order (fixed, part of the contract of the fixtures):
  1. Q  [B, H, 1, d]      N(0,1) fp32, seed `seed`
  2. K  [B, Hkv, S, d]    N(0,1) fp32, one batch element at a time
  3. V  [B, Hkv, S, d]    N(0,1) fp32, one batch element at a time
  4. per (b, kv head): `randperm(S_b)[:floor(plant_frac*S_b)]` positions, then
     noise N(0,1) [n, d]; K[b, g, pos] = 0.8 * q_mean[b, g] + 0.6 * noise where
     q_mean is the mean of the group's query heads.
Hash-MLP weights use a second generator seeded `seed + 1000`:
  for side in (k, q): for head: for layer: W [out, in] N(0, 1/fan_in), b [out] N(0, 0.01^2).
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np
import torch


@dataclass
class Workload:
    """One decode-step problem: post-RoPE Q/K/V of a single attention layer."""
    name: str
    batch: int
    seq_lens: List[int]               # per sequence context length (ragged allowed)
    n_q_heads: int = 32
    n_kv_heads: int = 8
    head_dim: int = 128
    n_code_heads: int = 8             # 32 = one K hash MLP per query head (reference-exact)
    lth_num_layers: int = 3
    lth_int_dim: int = 128
    lth_final_dim: int = 32
    init_budget: int = 128
    recent_budget: int = 128
    heavy_budget: float = 1.0 / 32
    dtype: torch.dtype = torch.bfloat16
    seed: int = 0
    plant_frac: float = 0.02

    @property
    def max_seq_len(self) -> int:
        return max(self.seq_lens)

    @property
    def code_words(self) -> int:
        return self.lth_final_dim // 32

    def heavy_count(self, s: int) -> int:
        # reference: hashattention/hashattention_llama.py:431-434
        hb = self.heavy_budget
        return int(hb) if hb > 1.0 else int(s * hb)

    def n_selected(self, s: int) -> int:
        ncand = max(0, s - self.init_budget - self.recent_budget)
        if ncand == 0:
            return s
        return min(self.init_budget, s) + min(self.heavy_count(s), ncand) + min(self.recent_budget, s)


def ragged_lengths_config4() -> List[int]:
    """Context lengths of the ragged workload: uniform in [8192, 131072], numpy seed 3."""
    return [int(x) for x in np.random.default_rng(3).integers(8192, 131073, 8)]


def named_workload(name: str) -> Workload:
    """The five benchmark/parity configurations."""
    if name == "config0":   # CPU-runnable, fp32, one K hash MLP per query head
        return Workload("config0", 1, [4096], n_code_heads=32, heavy_budget=0.25, dtype=torch.float32, seed=0)
    if name == "config1":
        return Workload("config1", 1, [32768], heavy_budget=1.0 / 8, seed=0)
    if name == "config2":   # headline: B=16, 64K context, 32x sparse
        return Workload("config2", 16, [65536] * 16, heavy_budget=1.0 / 32, seed=0)
    if name == "config3":   # per-layer share of the 32-layer decoder step
        return Workload("config3", 4, [131072] * 4, heavy_budget=1.0 / 32, seed=0)
    if name == "config4":   # ragged, 2-layer MLP, 64-bit codes
        return Workload("config4", 8, ragged_lengths_config4(), lth_num_layers=2, lth_final_dim=64,
                        heavy_budget=1.0 / 16, seed=3)
    raise KeyError(name)


@dataclass
class UsaWeights:
    """Hash-MLP parameters in `nn.Linear` convention (W [out, in], y = x W^T + b)."""
    k: List[List[tuple]] = field(default_factory=list)   # [head][layer] -> (W, b)
    q: List[List[tuple]] = field(default_factory=list)


def layer_dims(head_dim: int, int_dim: int, final_dim: int, num_layers: int):
    """(in, out) of every Linear of one hash MLP; reference hashattention_llama.py:99-128."""
    if num_layers == 3:
        return [(head_dim, int_dim), (int_dim, int_dim), (int_dim, final_dim)]
    if num_layers == 2:
        return [(head_dim, int_dim), (int_dim, final_dim)]
    if num_layers == 1:
        return [(head_dim, final_dim)]
    raise ValueError("lth_num_layers must be 1, 2 or 3")


def make_usa_weights(w: Workload, bias_std: float = 0.01) -> UsaWeights:
    g = torch.Generator().manual_seed(w.seed + 1000)
    dims = layer_dims(w.head_dim, w.lth_int_dim, w.lth_final_dim, w.lth_num_layers)
    out = UsaWeights()
    for side, n_heads in (("k", w.n_code_heads), ("q", w.n_q_heads)):
        heads = []
        for _ in range(n_heads):
            layers = []
            for (fi, fo) in dims:
                W = torch.randn(fo, fi, generator=g) * (fi ** -0.5)
                b = torch.randn(fo, generator=g) * bias_std
                layers.append((W, b))
            heads.append(layers)
        setattr(out, side, heads)
    return out


@dataclass
class Problem:
    w: Workload
    q: torch.Tensor        # [B, H, 1, d]
    k: torch.Tensor        # [B, Hkv, S_max, d]  (rows >= seq_len[b] are zero)
    v: torch.Tensor        # [B, Hkv, S_max, d]
    seq_lens: torch.Tensor  # int32 [B]
    usa: Optional[UsaWeights] = None


def make_problem(w: Workload, with_weights: bool = True) -> Problem:
    g = torch.Generator().manual_seed(w.seed)
    B, H, Hkv, d, S = w.batch, w.n_q_heads, w.n_kv_heads, w.head_dim, w.max_seq_len
    G = H // Hkv
    q = torch.randn(B, H, 1, d, generator=g)
    k = torch.zeros(B, Hkv, S, d, dtype=w.dtype)
    v = torch.zeros(B, Hkv, S, d, dtype=w.dtype)
    kf = []
    for b in range(B):
        kf.append(torch.randn(Hkv, w.seq_lens[b], d, generator=g))
    for b in range(B):
        v[b, :, : w.seq_lens[b]] = torch.randn(Hkv, w.seq_lens[b], d, generator=g).to(w.dtype)
    q_mean = q.view(B, Hkv, G, d).mean(dim=2)
    for b in range(B):
        sb = w.seq_lens[b]
        n_plant = int(w.plant_frac * sb)
        for hk in range(Hkv):
            pos = torch.randperm(sb, generator=g)[:n_plant]
            noise = torch.randn(n_plant, d, generator=g)
            kf[b][hk, pos] = 0.8 * q_mean[b, hk] + 0.6 * noise
        k[b, :, :sb] = kf[b].to(w.dtype)
        kf[b] = None
    return Problem(w, q.to(w.dtype), k, v, torch.tensor(w.seq_lens, dtype=torch.int32),
                   make_usa_weights(w) if with_weights else None)


def sha256_of(t: torch.Tensor) -> str:
    """Fingerprint of a tensor's raw bytes (bf16 viewed as int16)."""
    t = t.detach().contiguous().cpu()
    if t.dtype == torch.bfloat16:
        t = t.view(torch.int16)
    return hashlib.sha256(t.numpy().tobytes()).hexdigest()


def make_problem_on_device(w: Workload, device="cuda:0", with_weights: bool = True) -> Problem:
    """Same recipe as `make_problem` drawn with the device generator: the distribution is identical, the
    bytes are not (use `make_problem` wherever bytes must match fixtures).  Built one sequence at a time
    so the full-size workloads never hold an fp32 copy of the whole cache."""
    g = torch.Generator(device=device).manual_seed(w.seed)
    B, H, Hkv, d, S = w.batch, w.n_q_heads, w.n_kv_heads, w.head_dim, w.max_seq_len
    G = H // Hkv
    q = torch.randn(B, H, 1, d, generator=g, device=device)
    k = torch.zeros(B, Hkv, S, d, dtype=w.dtype, device=device)
    v = torch.zeros(B, Hkv, S, d, dtype=w.dtype, device=device)
    q_mean = q.view(B, Hkv, G, d).mean(dim=2)
    for b in range(B):
        sb = w.seq_lens[b]
        kb = torch.randn(Hkv, sb, d, generator=g, device=device)
        n_plant = int(w.plant_frac * sb)
        for hk in range(Hkv):
            pos = torch.randperm(sb, generator=g, device=device)[:n_plant]
            kb[hk, pos] = 0.8 * q_mean[b, hk] + 0.6 * torch.randn(n_plant, d, generator=g, device=device)
        k[b, :, :sb] = kb.to(w.dtype)
        v[b, :, :sb] = torch.randn(Hkv, sb, d, generator=g, device=device).to(w.dtype)
        del kb
    return Problem(w, q.to(w.dtype), k, v, torch.tensor(w.seq_lens, dtype=torch.int32, device=device),
                   make_usa_weights(w) if with_weights else None)
