"""ctypes binding of libhashattn.so (the C ABI declared in include/hashattn.h).

Every wrapper takes torch tensors that already live on the GPU, passes raw pointers, sizes and
the current HIP stream, and raises `HashAttnError` on a non-zero status.  There is no CPU
fallback: without the built library, or without a GPU, the calls fail loudly.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Tuple

import torch

_LIB_NAME = "libhashattn.so"
_lib = None

HA_F32, HA_BF16, HA_F16 = 0, 1, 2
HA_ARITH_F32, HA_ARITH_BF16 = 0, 1
HA_SELECT_SIMPLE, HA_SELECT_THRESHOLD = 0, 1
HA_SELECT_ALGO_AUTO, HA_SELECT_ALGO_HISTOGRAM, HA_SELECT_ALGO_SAMPLED, HA_SELECT_ALGO_SAMPLED_EXACT_ROWS = 0, 1, 2, 3

_DTYPE = {torch.float32: HA_F32, torch.bfloat16: HA_BF16, torch.float16: HA_F16}


class HashAttnError(RuntimeError):
    def __init__(self, status: int, where: str, detail: str):
        self.status = status
        super().__init__(f"{where} failed with status {status}: {detail}")


def lib_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


def load_library() -> C.CDLL:
    """Load the built library once; raise if it has not been built (no silent fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python hashattention-1.0_amd/build.py` "
                          "(hipcc --offload-arch=gfx950); there is no CPU fallback")
    _lib = _declare(C.CDLL(path))
    return _lib


def load_wait_all_variant() -> C.CDLL:
    """The library's twin built with -DHASHATTN_STAGE_WAIT_ALL (tests compare the two builds bit for bit); not cached."""
    path = os.path.join(os.path.dirname(lib_path()), "libhashattn_waitall.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: `python hashattention-1.0_amd/build.py` builds it next to the library")
    return _declare(C.CDLL(path))


def _declare(lib: C.CDLL) -> C.CDLL:
    """Argument and result types of every entry point of include/hashattn.h on a loaded library."""
    vp, i32, i64, f32, f64, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_double, C.c_size_t
    lib.ha_version.restype = i32
    lib.ha_status_string.restype = C.c_char_p
    lib.ha_status_string.argtypes = [i32]
    lib.ha_last_error_string.restype = C.c_char_p
    lib.ha_device_count.restype = i32
    lib.ha_usa_packed_floats.restype = i64
    lib.ha_usa_packed_floats.argtypes = [i32, i32, i32, i32]
    lib.ha_encode_pack.restype = i32
    lib.ha_encode_pack.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i32, i32, i32, i32, i32,
                                   vp, i64, i64, i32, vp, vp, vp]
    lib.ha_encode_step.restype = i32
    lib.ha_encode_step.argtypes = [vp, i64, i64, i64, vp, i64, i64, i32, i32, i32, i32, i32, i32, vp, vp,
                                   i32, i32, i32, i32, i32, vp, i64, i64, i32, vp, vp, vp]
    lib.ha_encode_step_cached.restype = i32
    lib.ha_encode_step_cached.argtypes = [vp, i64, i64, i64, vp, i64, i64, i32, i32, i32, i32, i32, vp, vp, vp,
                                          i32, i32, i32, i32, i32, vp, i64, i64, vp, vp]
    lib.ha_encode_pack_prefill.restype = i32
    lib.ha_encode_pack_prefill.argtypes = [vp, i64, i64, i64, i32, i32, i32, i32, vp, i32, i32, i32, i32,
                                           vp, i64, i64, i32, vp, vp]
    lib.ha_encode_pack_prefill_f32.restype = i32
    lib.ha_encode_pack_prefill_f32.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i32, i32, i32, i32,
                                               vp, i64, i64, i32, vp, vp]
    lib.ha_hamming_score.restype = i32
    lib.ha_hamming_score.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, vp, vp, vp]
    lib.ha_select_workspace_bytes.restype = sz
    lib.ha_select_workspace_bytes.argtypes = [i32, i32, i32, i32, i32]
    lib.ha_select.restype = i32
    lib.ha_select.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, vp, i32, i32, f64, i32, i32, i32,
                              vp, i64, vp, vp, sz, vp]
    lib.ha_select_rows.restype = i32
    lib.ha_select_rows.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, i32, vp, i32, i32, f64, i32, i32, vp, i64, vp, vp, sz, vp]
    lib.ha_sparse_decode_rows.restype = i32
    lib.ha_sparse_decode_rows.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i64, vp, f32,
                                          vp, i64, i32, vp, vp, sz, vp]
    lib.ha_select_static_max_bytes.restype = sz
    lib.ha_select_static.restype = i32
    lib.ha_select_static.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, vp, i32, i32, f64, i32, i32, vp, i64, vp, vp]
    lib.ha_rope_append.restype = i32
    lib.ha_rope_append.argtypes = [vp, i64, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp]
    lib.ha_rope_encode_step.restype = i32
    lib.ha_rope_encode_step.argtypes = [vp, i64, i32, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp, vp,
                                        i32, i32, i32, i32, i32, vp, i64, i64, vp, vp]
    lib.ha_rope_encode_step_cos_sin.restype = i32
    lib.ha_rope_encode_step_cos_sin.argtypes = [vp, i64, i32, i32, i32, i32, i32, i32, vp, vp, vp, i64, vp, vp, vp, i64, i64, i64, i64, vp, vp,
                                                i32, i32, i32, i32, i32, vp, i64, i64, vp, vp]
    lib.ha_linear_skinny.restype = i32
    lib.ha_linear_skinny.argtypes = [vp, i64, vp, i64, vp, i64, vp, i64, i32, i32, i32, vp]
    lib.ha_linear_skinny_fused.restype = i32
    lib.ha_linear_skinny_fused.argtypes = [vp, i64, vp, i64, vp, i64, vp, C.c_float, i32, vp, i64, i32, i32, i32, vp]
    lib.ha_swiglu.restype = i32
    lib.ha_swiglu.argtypes = [vp, i64, i32, i32, i32, vp, vp]
    lib.ha_select_prepare.restype = i32
    lib.ha_select_prepare.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, vp, i32, i32, f64, i32, i32, vp, vp, sz, vp]
    lib.ha_select_histogram.restype = i32
    lib.ha_select_histogram.argtypes = [vp, i64, i64, vp, i32, i32, i32, i32, i32, vp, i32, i32, vp, sz, vp]
    lib.ha_sparse_decode_fused_local_thresholds.restype = i32
    lib.ha_sparse_decode_fused_local_thresholds.argtypes = [i32, i32, i32]
    lib.ha_sparse_decode_fused_applies.restype = i32
    lib.ha_sparse_decode_fused_applies.argtypes = [i32, i32, i32, i32, i32, i32, i32, f64, i32]
    lib.ha_sparse_decode_fused_workspace_bytes.restype = sz
    lib.ha_sparse_decode_fused_workspace_bytes.argtypes = [i32, i32, i32, i32]
    lib.ha_sparse_decode_fused.restype = i32
    lib.ha_sparse_decode_fused.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, vp, i64, i64, vp, i32, i32, i32, i32, i32, i32, vp,
                                           i32, i32, f64, vp, sz, i32, vp, f32, vp, vp, sz, vp]
    lib.ha_sparse_decode_workspace_bytes.restype = sz
    lib.ha_sparse_decode_workspace_bytes.argtypes = [i32, i32, i64]
    lib.ha_sparse_decode.restype = i32
    lib.ha_sparse_decode.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, vp, i64, vp, f32,
                                     vp, vp, sz, vp]
    lib.ha_sparse_decode_masked.restype = i32
    lib.ha_sparse_decode_masked.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, vp, i64, vp, f32,
                                            vp, i64, i32, i32, vp, vp, sz, vp]
    lib.ha_sparse_decode_paged.restype = i32
    lib.ha_sparse_decode_paged.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i64, vp, f32,
                                           vp, i64, i32, i32, vp, i64, i64, vp, vp, sz, vp]
    lib.ha_sparse_decode_fused_paged.restype = i32
    lib.ha_sparse_decode_fused_paged.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, vp, i64, i64, vp, i32, i32, i32, i32, i32, i32,
                                                 vp, i32, i32, f64, vp, sz, i32, vp, vp, i64, i64, f32, vp, vp, sz, vp]
    lib.ha_sparse_decode_fused_prefix_masked.restype = i32
    lib.ha_sparse_decode_fused_prefix_masked.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, vp, i64, i64, vp, i32, i32, i32, i32,
                                                         i32, i32, vp, i32, i32, f64, vp, sz, i32, vp, vp, f32, vp, vp, sz, vp]
    lib.ha_weight_tiles_elems.restype = i64
    lib.ha_weight_tiles_elems.argtypes = [i32, i32, i32]
    lib.ha_pack_weight_tiles.restype = i32
    lib.ha_pack_weight_tiles.argtypes = [vp, i64, i32, i32, i32, vp, vp]
    lib.ha_linear_tiled.restype = i32
    lib.ha_linear_tiled.argtypes = [vp, i64, vp, vp, i64, i32, vp, i64, i32, i32, i32, vp]
    lib.ha_rmsnorm.restype = i32
    lib.ha_rmsnorm.argtypes = [vp, i64, vp, i32, i32, i32, f32, vp, i64, vp]
    lib.ha_window_partial_bytes.restype = sz
    lib.ha_window_partial_bytes.argtypes = [i32, i32]
    lib.ha_window_partial.restype = i32
    lib.ha_window_partial.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i32, i32, f32, vp, vp]
    lib.ha_sparse_decode_heavy.restype = i32
    lib.ha_sparse_decode_heavy.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, vp, i64, vp, f32,
                                           vp, vp, sz, vp, i32, i32, i32, vp, vp]
    lib.ha_dense_decode_workspace_bytes.restype = sz
    lib.ha_dense_decode_workspace_bytes.argtypes = [i32, i32, i32]
    lib.ha_dense_decode.restype = i32
    lib.ha_dense_decode.argtypes = [vp, i64, i64, vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, f32,
                                    vp, vp, sz, vp]
    return lib


def _check(status: int, where: str):
    if status != 0:
        raise HashAttnError(status, where, load_library().ha_last_error_string().decode())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor):
    """The current stream of t's device as the hipStream_t the library takes.  Through torch's raw-handle accessor where
    there is one: building a `torch.cuda.Stream` object per launch costs ~5 us, a fifth of what a decode layer's launches
    cost the host."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)          # a plain integer: ctypes turns it into the void * the signature asks for
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("hashattention ops take GPU tensors only (there is no CPU path)")


def workspace(nbytes: int, device) -> torch.Tensor:
    """A byte buffer of at least nbytes (torch's allocator returns >= 256-byte aligned blocks)."""
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------------------ encode

def pack_usa_weights(layers_per_head, device=None) -> torch.Tensor:
    """[[(W [out,in], b [out]), ...] per head] -> fp32 blob [n_heads, per_head]: per layer W then b.  W is stored
    transposed with its inputs in groups of four, [in / 4][out][4], when `in` is a multiple of 16 (the 128-bit
    coalesced fetch of the encode kernels), as plain W^T [in][out] otherwise."""
    blobs = []
    for layers in layers_per_head:
        parts = []
        for (W, b) in layers:
            wt = W.detach().float().t().contiguous()                      # [in, out]
            if wt.shape[0] % 16 == 0:
                wt = wt.view(wt.shape[0] // 4, 4, wt.shape[1]).permute(0, 2, 1).contiguous()
            parts.append(wt.reshape(-1))
            parts.append(b.detach().float().reshape(-1))
        blobs.append(torch.cat(parts))
    out = torch.stack(blobs).contiguous()
    return out.to(device) if device is not None else out


def pack_usa_weights_bf16(layers_per_head, device=None) -> torch.Tensor:
    """Blob for the MFMA encoder: per layer W [out][in] (native nn.Linear orientation) then b, in bf16."""
    blobs = []
    for layers in layers_per_head:
        parts = []
        for (W, b) in layers:
            parts.append(W.detach().to(torch.bfloat16).contiguous().reshape(-1))
            parts.append(b.detach().to(torch.bfloat16).reshape(-1))
        blobs.append(torch.cat(parts))
    out = torch.stack(blobs).contiguous()
    return out.to(device) if device is not None else out


def encode_pack(x: torch.Tensor, weights: torch.Tensor, n_layers: int, int_dim: int, final_dim: int,
                codes: torch.Tensor, pos0: int = 0, pos_dev: Optional[torch.Tensor] = None,
                arith: int = HA_ARITH_F32, want_logits: bool = False) -> Optional[torch.Tensor]:
    """x [B, x_heads, T, d]; weights [n_heads, per_head] fp32; codes [B, n_heads, S_cap, W] int32 (written in place)."""
    _require_cuda(x, weights, codes, pos_dev)
    lib = load_library()
    B, xh, T, d = x.shape
    n_heads = weights.shape[0]
    assert x.stride(3) == 1 and codes.stride(3) == 1 and codes.stride(2) == codes.shape[3]
    assert codes.shape[0] >= B and codes.shape[1] == n_heads, "codes must be [>= B, n_heads, ., W] for x [B, ., T, d]"
    assert codes.dtype == torch.int32 and weights.dtype == torch.float32 and weights.is_contiguous()
    assert weights.shape[1] == lib.ha_usa_packed_floats(n_layers, d, int_dim, final_dim)
    if pos_dev is None:
        assert pos0 + T <= codes.shape[2]
    logits = torch.empty(B, n_heads, T, final_dim, dtype=torch.float32, device=x.device) if want_logits else None
    _check(lib.ha_encode_pack(_ptr(x), _DTYPE[x.dtype], x.stride(0), x.stride(1), x.stride(2), B, xh, n_heads, T,
                              _ptr(weights), n_layers, d, int_dim, final_dim, arith,
                              _ptr(codes), codes.stride(0), codes.stride(1), pos0, _ptr(pos_dev), _ptr(logits), _stream(x)),
           "ha_encode_pack")
    return logits


def encode_step(k_new: torch.Tensor, q3: torch.Tensor, wk: torch.Tensor, wq: torch.Tensor, n_layers: int, int_dim: int,
                final_dim: int, kcodes: torch.Tensor, qcodes: torch.Tensor, pos0: int = 0,
                pos_dev: Optional[torch.Tensor] = None, arith: int = HA_ARITH_F32) -> None:
    """One launch for a decode step: k_new [B, Hkv, 1, d] appended to kcodes at pos0 / pos_dev[b]; q3 [B, H, d] -> qcodes [B, H, W]."""
    _require_cuda(k_new, q3, wk, wq, kcodes, qcodes, pos_dev)
    lib = load_library()
    B, Hkv, T, d = k_new.shape
    H = q3.shape[1]
    assert T == 1 and k_new.stride(3) == 1 and q3.stride(2) == 1 and k_new.dtype == q3.dtype
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == kcodes.shape[3] and qcodes.is_contiguous()
    assert kcodes.dtype == torch.int32 and qcodes.dtype == torch.int32 and qcodes.numel() == B * H * (final_dim // 32)
    _check(lib.ha_encode_step(_ptr(k_new), k_new.stride(0), k_new.stride(1), k_new.stride(2), _ptr(q3), q3.stride(0), q3.stride(1),
                              _DTYPE[k_new.dtype], B, Hkv, wk.shape[0], H, 1, _ptr(wk), _ptr(wq), n_layers, d, int_dim, final_dim,
                              arith, _ptr(kcodes), kcodes.stride(0), kcodes.stride(1), pos0, _ptr(pos_dev), _ptr(qcodes),
                              _stream(q3)), "ha_encode_step")


def encode_step_cached(k_cache: torch.Tensor, q3: torch.Tensor, wk: torch.Tensor, wq: torch.Tensor, n_layers: int, int_dim: int,
                       final_dim: int, kcodes: torch.Tensor, qcodes: torch.Tensor, seq_lens: torch.Tensor,
                       arith: int = HA_ARITH_F32) -> None:
    """`encode_step` for lengths on the device: the newest key of sequence b is row seq_lens[b] - 1 of k_cache [B, Hkv, S_cap, d],
    its code goes to the same position of kcodes; q3 [B, H, d] -> qcodes [B, H, W]."""
    _require_cuda(k_cache, q3, wk, wq, kcodes, qcodes, seq_lens)
    lib = load_library()
    B, Hkv, _, d = k_cache.shape
    H = q3.shape[1]
    assert k_cache.stride(3) == 1 and q3.stride(2) == 1 and k_cache.dtype == q3.dtype
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == kcodes.shape[3] and qcodes.is_contiguous()
    assert kcodes.dtype == torch.int32 and qcodes.dtype == torch.int32 and qcodes.numel() == B * H * (final_dim // 32)
    assert seq_lens.dtype == torch.int32 and seq_lens.numel() == B and seq_lens.is_contiguous()
    _check(lib.ha_encode_step_cached(_ptr(k_cache), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), _ptr(q3), q3.stride(0),
                                     q3.stride(1), _DTYPE[k_cache.dtype], B, Hkv, wk.shape[0], H, _ptr(seq_lens), _ptr(wk), _ptr(wq),
                                     n_layers, d, int_dim, final_dim, arith, _ptr(kcodes), kcodes.stride(0), kcodes.stride(1),
                                     _ptr(qcodes), _stream(q3)), "ha_encode_step_cached")


def encode_pack_prefill(x: torch.Tensor, weights_bf16: torch.Tensor, n_layers: int, int_dim: int, final_dim: int,
                        codes: torch.Tensor, pos0: int = 0, pos_dev: Optional[torch.Tensor] = None) -> None:
    """bf16 MFMA bulk encode; same tensor conventions as `encode_pack`, weights from `pack_usa_weights_bf16`."""
    _require_cuda(x, weights_bf16, codes, pos_dev)
    lib = load_library()
    B, xh, T, d = x.shape
    n_heads = weights_bf16.shape[0]
    assert x.dtype == torch.bfloat16 and weights_bf16.dtype == torch.bfloat16 and weights_bf16.is_contiguous()
    assert x.stride(3) == 1 and codes.stride(3) == 1 and codes.stride(2) == codes.shape[3] and codes.dtype == torch.int32
    assert codes.shape[0] >= B and codes.shape[1] == n_heads, "codes must be [>= B, n_heads, ., W] for x [B, ., T, d]"
    if pos_dev is None:
        assert pos0 + T <= codes.shape[2]
    _check(lib.ha_encode_pack_prefill(_ptr(x), x.stride(0), x.stride(1), x.stride(2), B, xh, n_heads, T,
                                      _ptr(weights_bf16), n_layers, d, int_dim, final_dim,
                                      _ptr(codes), codes.stride(0), codes.stride(1), pos0, _ptr(pos_dev), _stream(x)),
           "ha_encode_pack_prefill")


def encode_pack_prefill_f32(x: torch.Tensor, weights: torch.Tensor, n_layers: int, int_dim: int, final_dim: int,
                            codes: torch.Tensor, pos0: int = 0, pos_dev: Optional[torch.Tensor] = None) -> None:
    """fp32 MFMA bulk encode for fp32 hash modules; tensors as `encode_pack` (weights from `pack_usa_weights`)."""
    _require_cuda(x, weights, codes, pos_dev)
    lib = load_library()
    B, xh, T, d = x.shape
    n_heads = weights.shape[0]
    assert weights.dtype == torch.float32 and weights.is_contiguous()
    assert weights.shape[1] == lib.ha_usa_packed_floats(n_layers, d, int_dim, final_dim)
    assert x.stride(3) == 1 and codes.stride(3) == 1 and codes.stride(2) == codes.shape[3] and codes.dtype == torch.int32
    assert codes.shape[0] >= B and codes.shape[1] == n_heads, "codes must be [>= B, n_heads, ., W] for x [B, ., T, d]"
    if pos_dev is None:
        assert pos0 + T <= codes.shape[2]
    _check(lib.ha_encode_pack_prefill_f32(_ptr(x), _DTYPE[x.dtype], x.stride(0), x.stride(1), x.stride(2), B, xh, n_heads, T,
                                          _ptr(weights), n_layers, d, int_dim, final_dim,
                                          _ptr(codes), codes.stride(0), codes.stride(1), pos0, _ptr(pos_dev), _stream(x)),
           "ha_encode_pack_prefill_f32")


# ------------------------------------------------------------------------------------------ score / select

def hamming_score(kcodes: torch.Tensor, qcodes: torch.Tensor, max_seq_len: int,
                  seq_lens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """kcodes [B, Hc, S_cap, W] int32, qcodes [B, H, W] int32 -> uint8 [B, H, max_seq_len] (rows >= seq_len are 255)."""
    _require_cuda(kcodes, qcodes, seq_lens)
    lib = load_library()
    B, Hc, _, W = kcodes.shape
    H = qcodes.shape[1]
    assert qcodes.is_contiguous() and kcodes.stride(3) == 1 and kcodes.stride(2) == W
    scores = torch.full((B, H, max_seq_len), 255, dtype=torch.uint8, device=kcodes.device)
    _check(lib.ha_hamming_score(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H, Hc, W, max_seq_len,
                                _ptr(seq_lens), _ptr(scores), _stream(kcodes)), "ha_hamming_score")
    return scores


def select_workspace_bytes(B, H, Hc, W, max_seq_len) -> int:
    return load_library().ha_select_workspace_bytes(B, H, Hc, W, max_seq_len)


def select(kcodes: torch.Tensor, qcodes: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
           init_budget: int, recent_budget: int, heavy_budget: float, out_idx: torch.Tensor, out_counts: torch.Tensor,
           ws: torch.Tensor, mode: int = HA_SELECT_SIMPLE, depth: int = 0, algo: int = HA_SELECT_ALGO_AUTO) -> None:
    """Ascending index lists out_idx [B, H, idx_cap] int32 and out_counts [B, H] int32 (both written in place)."""
    _require_cuda(kcodes, qcodes, seq_lens, out_idx, out_counts, ws)
    lib = load_library()
    B, Hc, _, W = kcodes.shape
    H = qcodes.shape[1]
    assert qcodes.is_contiguous() and kcodes.stride(3) == 1 and kcodes.stride(2) == W
    assert out_idx.is_contiguous() and out_idx.dtype == torch.int32 and out_counts.is_contiguous() and out_counts.dtype == torch.int32
    assert seq_lens is None or (seq_lens.dtype == torch.int32 and seq_lens.is_contiguous())
    _check(lib.ha_select(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H, Hc, W, max_seq_len,
                         _ptr(seq_lens), init_budget, recent_budget, float(heavy_budget), mode, depth, algo,
                         _ptr(out_idx), out_idx.shape[2], _ptr(out_counts), _ptr(ws), ws.numel(), _stream(kcodes)), "ha_select")


def select_rows(kcodes: torch.Tensor, qcodes: torch.Tensor, rows_per_sequence: int, max_seq_len: int, seq_lens: torch.Tensor,
                init_budget: int, recent_budget: int, heavy_budget: float, out_idx: torch.Tensor, out_counts: torch.Tensor,
                ws: torch.Tensor, mode: int = HA_SELECT_SIMPLE, depth: int = 0) -> None:
    """`select` for chunks of tokens: qcodes [n_rows, H, W], seq_lens [n_rows], lists [n_rows, H, cap]; row n is a query
    against the codes of sequence n // rows_per_sequence (kcodes [n_seq, Hc, S_cap, W])."""
    _require_cuda(kcodes, qcodes, seq_lens, out_idx, out_counts, ws)
    lib = load_library()
    n_seq, Hc, _, W = kcodes.shape
    n_rows, H = qcodes.shape[0], qcodes.shape[1]
    assert n_rows == n_seq * rows_per_sequence and qcodes.is_contiguous() and kcodes.stride(3) == 1 and kcodes.stride(2) == W
    assert out_idx.is_contiguous() and out_idx.dtype == torch.int32 and out_counts.is_contiguous() and out_counts.dtype == torch.int32
    assert out_idx.shape[0] == n_rows and seq_lens.dtype == torch.int32 and seq_lens.is_contiguous() and seq_lens.numel() == n_rows
    _check(lib.ha_select_rows(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), n_rows, rows_per_sequence, H, Hc, W,
                              max_seq_len, _ptr(seq_lens), init_budget, recent_budget, float(heavy_budget), mode, depth,
                              _ptr(out_idx), out_idx.shape[2], _ptr(out_counts), _ptr(ws), ws.numel(), _stream(kcodes)), "ha_select_rows")


def sparse_decode_rows(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, rows_per_sequence: int, idx: torch.Tensor,
                       counts: torch.Tensor, sm_scale: float, out: torch.Tensor, ws: torch.Tensor,
                       mask: Optional[torch.Tensor] = None) -> None:
    """`sparse_decode` for chunks of tokens: q, out [n_rows, H, 128], idx [n_rows, H, cap]; row n attends to the cache of
    sequence n // rows_per_sequence (k, v [n_seq, Hkv, S_cap, 128]).  mask: optional fp32 [n_rows, n], by token position."""
    _require_cuda(q, k, v, idx, counts, out, ws, mask)
    lib = load_library()
    n_rows, H, _ = q.shape
    assert n_rows == k.shape[0] * rows_per_sequence and out.is_contiguous() and out.dtype == q.dtype and out.shape == q.shape
    assert idx.is_contiguous() and counts.is_contiguous() and idx.shape[0] == n_rows
    if mask is not None:
        assert mask.dtype == torch.float32 and mask.dim() == 2 and mask.shape[0] == n_rows and mask.stride(1) == 1
    _check(lib.ha_sparse_decode_rows(*_kv_args(q, k, v), n_rows, rows_per_sequence, H, k.shape[1], _ptr(idx), idx.shape[2], _ptr(counts),
                                     float(sm_scale), _ptr(mask), mask.stride(0) if mask is not None else 0,
                                     mask.shape[1] if mask is not None else 0, _ptr(out), _ptr(ws), ws.numel(), _stream(q)),
           "ha_sparse_decode_rows")


def select_static(kcodes: torch.Tensor, qcodes: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
                  init_budget: int, recent_budget: int, heavy_budget: float, out_idx: torch.Tensor, out_counts: torch.Tensor,
                  mode: int = HA_SELECT_SIMPLE, depth: int = 0) -> None:
    """`select` without a workspace: the library's built-in device scratch is used and nothing is allocated (shapes whose
    scratch exceeds ha_select_static_max_bytes() are refused).  Calls on one GPU must not overlap in time."""
    _require_cuda(kcodes, qcodes, seq_lens, out_idx, out_counts)
    lib = load_library()
    B, Hc, _, W = kcodes.shape
    H = qcodes.shape[1]
    assert qcodes.is_contiguous() and kcodes.stride(3) == 1 and kcodes.stride(2) == W
    assert out_idx.is_contiguous() and out_idx.dtype == torch.int32 and out_counts.is_contiguous() and out_counts.dtype == torch.int32
    assert seq_lens is None or (seq_lens.dtype == torch.int32 and seq_lens.is_contiguous())
    _check(lib.ha_select_static(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H, Hc, W, max_seq_len,
                                _ptr(seq_lens), init_budget, recent_budget, float(heavy_budget), mode, depth,
                                _ptr(out_idx), out_idx.shape[2], _ptr(out_counts), _stream(kcodes)), "ha_select_static")


def select_prepare(kcodes: torch.Tensor, qcodes: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
                   init_budget: int, recent_budget: int, heavy_budget: float, out_counts: torch.Tensor, ws: torch.Tensor,
                   mode: int = HA_SELECT_SIMPLE, depth: int = 0) -> None:
    """Thresholds and per-chunk offsets into the workspace, counts into out_counts [B, H]: the first half of the fused path."""
    _require_cuda(kcodes, qcodes, seq_lens, out_counts, ws)
    lib = load_library()
    B, Hc, _, W = kcodes.shape
    H = qcodes.shape[1]
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == W and qcodes.is_contiguous() and out_counts.is_contiguous()
    _check(lib.ha_select_prepare(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H, Hc, W, max_seq_len,
                                 _ptr(seq_lens), init_budget, recent_budget, float(heavy_budget), mode, depth, _ptr(out_counts),
                                 _ptr(ws), ws.numel(), _stream(kcodes)), "ha_select_prepare")


def select_histogram(kcodes: torch.Tensor, qcodes: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
                     init_budget: int, recent_budget: int, ws: torch.Tensor) -> None:
    """Per-chunk distance histograms into the workspace: all the fused attention launch needs when it derives the
    thresholds itself (sparse_decode_fused(..., thresholds_ready=False))."""
    _require_cuda(kcodes, qcodes, seq_lens, ws)
    lib = load_library()
    B, Hc, _, W = kcodes.shape
    H = qcodes.shape[1]
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == W and qcodes.is_contiguous()
    _check(lib.ha_select_histogram(_ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H, Hc, W, max_seq_len,
                                   _ptr(seq_lens), init_budget, recent_budget, _ptr(ws), ws.numel(), _stream(kcodes)),
           "ha_select_histogram")


def fused_local_thresholds(B, Hc, max_seq_len) -> bool:
    return bool(load_library().ha_sparse_decode_fused_local_thresholds(B, Hc, max_seq_len))


def fused_applies(B, H, Hc, W, max_seq_len, init_budget, recent_budget, heavy_budget, mode=HA_SELECT_SIMPLE) -> bool:
    return bool(load_library().ha_sparse_decode_fused_applies(B, H, Hc, W, max_seq_len, init_budget, recent_budget,
                                                              float(heavy_budget), mode))


def sparse_decode_fused_workspace_bytes(B, H, Hc, max_seq_len) -> int:
    return load_library().ha_sparse_decode_fused_workspace_bytes(B, H, Hc, max_seq_len)


def _slot_args(slots: torch.Tensor, n_seq: int, n_slots: int):
    """slots int32 [n_seq, >= S] (or [1, .] expanded: row stride 0): the K/V row of token j of sequence b is row slots[b, j]."""
    assert slots.dtype == torch.int32 and slots.dim() == 2 and slots.shape[0] == n_seq and slots.stride(1) == 1
    return (_ptr(slots), slots.stride(0), int(n_slots))


def sparse_decode_fused(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kcodes: torch.Tensor, qcodes: torch.Tensor,
                        max_seq_len: int, seq_lens: Optional[torch.Tensor], init_budget: int, recent_budget: int,
                        heavy_budget: float, ws_select: torch.Tensor, sm_scale: float, out: torch.Tensor, ws: torch.Tensor,
                        thresholds_ready: bool = True, out_counts: Optional[torch.Tensor] = None,
                        slots: Optional[torch.Tensor] = None, masked_prefix: Optional[torch.Tensor] = None) -> None:
    """Attention over the selection prepared by select_prepare (same codes, budgets and seq_lens); out [B,H,128] in place.
    thresholds_ready=False: the workspace was filled by select_histogram only; counts (optional, [B,H] int32) are written here.
    slots: optional token -> slot table int32 [B, >= max_seq_len] of a paged cache; k, v are then [B or 1 (expanded), Hkv,
    n_slots, 128] views of the row pool (`ha_sparse_decode_fused_paged`).
    masked_prefix: optional int32 [B]: tokens below masked_prefix[b] score -inf, the mask of a left-padded batch
    (`ha_sparse_decode_fused_prefix_masked`)."""
    _require_cuda(q, k, v, kcodes, qcodes, seq_lens, ws_select, out, ws, out_counts, slots, masked_prefix)
    lib = load_library()
    B, H, _ = q.shape
    Hc, W = kcodes.shape[1], kcodes.shape[3]
    assert out.is_contiguous() and out.dtype == q.dtype and kcodes.stride(3) == 1 and kcodes.stride(2) == W and qcodes.is_contiguous()
    if masked_prefix is not None:
        assert slots is None and masked_prefix.dtype == torch.int32 and masked_prefix.is_contiguous() and masked_prefix.numel() == B
        _check(lib.ha_sparse_decode_fused_prefix_masked(*_kv_args(q, k, v), _ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes),
                                                        B, H, k.shape[1], Hc, W, max_seq_len, _ptr(seq_lens), init_budget, recent_budget,
                                                        float(heavy_budget), _ptr(ws_select), ws_select.numel(),
                                                        1 if thresholds_ready else 0, _ptr(out_counts), _ptr(masked_prefix),
                                                        float(sm_scale), _ptr(out), _ptr(ws), ws.numel(), _stream(q)),
               "ha_sparse_decode_fused_prefix_masked")
        return
    if slots is not None:
        assert slots.shape[1] >= max_seq_len
        _check(lib.ha_sparse_decode_fused_paged(*_kv_args(q, k, v), _ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H,
                                                k.shape[1], Hc, W, max_seq_len, _ptr(seq_lens), init_budget, recent_budget,
                                                float(heavy_budget), _ptr(ws_select), ws_select.numel(), 1 if thresholds_ready else 0,
                                                _ptr(out_counts), *_slot_args(slots, B, k.shape[2]), float(sm_scale), _ptr(out), _ptr(ws),
                                                ws.numel(), _stream(q)), "ha_sparse_decode_fused_paged")
        return
    _check(lib.ha_sparse_decode_fused(*_kv_args(q, k, v), _ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes), B, H,
                                      k.shape[1], Hc, W, max_seq_len, _ptr(seq_lens), init_budget, recent_budget, float(heavy_budget),
                                      _ptr(ws_select), ws_select.numel(), 1 if thresholds_ready else 0, _ptr(out_counts),
                                      float(sm_scale), _ptr(out), _ptr(ws), ws.numel(), _stream(q)), "ha_sparse_decode_fused")


# ------------------------------------------------------------------------------------------ attention

def sparse_decode_workspace_bytes(B, H, idx_cap) -> int:
    return load_library().ha_sparse_decode_workspace_bytes(B, H, idx_cap)


def _kv_args(q, k, v):
    assert q.dim() == 3 and k.dim() == 4 and v.shape == k.shape and v.stride() == k.stride()
    assert q.stride(2) == 1 and k.stride(3) == 1 and q.dtype == k.dtype == v.dtype
    return (_ptr(q), q.stride(0), q.stride(1), _ptr(k), _ptr(v), _DTYPE[k.dtype], k.stride(0), k.stride(1), k.stride(2))


def sparse_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor, counts: torch.Tensor,
                  sm_scale: float, out: torch.Tensor, ws: torch.Tensor, mask: Optional[torch.Tensor] = None,
                  mask_by_slot: bool = False, slots: Optional[torch.Tensor] = None, rows_per_sequence: int = 1) -> None:
    """q [B,H,128]; k,v [B,Hkv,S_cap,128]; idx [B,H,idx_cap] int32; counts [B,H] int32; out [B,H,128] (in place).
    mask: optional fp32 [B, n] (or [1, n] expanded: row stride 0) added to the scaled scores, indexed by token position,
    or by the place in the list when mask_by_slot.
    slots: optional token -> slot table int32 [n_seq, >= S] of a paged cache (`ha_sparse_decode_paged`): k, v are then
    [n_seq or 1 (expanded), Hkv, n_slots, 128] views of the row pool; n_seq = B // rows_per_sequence."""
    _require_cuda(q, k, v, idx, counts, out, ws, mask, slots)
    lib = load_library()
    B, H, _ = q.shape
    assert out.is_contiguous() and out.dtype == q.dtype and idx.is_contiguous() and counts.is_contiguous()
    if slots is not None:
        assert B % rows_per_sequence == 0
        if mask is not None:
            assert mask.dtype == torch.float32 and mask.dim() == 2 and mask.shape[0] == B and mask.stride(1) == 1
        _check(lib.ha_sparse_decode_paged(*_kv_args(q, k, v), B, rows_per_sequence, H, k.shape[1], _ptr(idx), idx.shape[2], _ptr(counts),
                                          float(sm_scale), _ptr(mask), mask.stride(0) if mask is not None else 0,
                                          mask.shape[1] if mask is not None else 0, 1 if mask_by_slot else 0,
                                          *_slot_args(slots, B // rows_per_sequence, k.shape[2]), _ptr(out), _ptr(ws), ws.numel(),
                                          _stream(q)), "ha_sparse_decode_paged")
        return
    assert rows_per_sequence == 1, "chunks of rows without a slot table go through sparse_decode_rows"
    if mask is not None:
        assert mask.dtype == torch.float32 and mask.dim() == 2 and mask.shape[0] == B and mask.stride(1) == 1
        _check(lib.ha_sparse_decode_masked(*_kv_args(q, k, v), B, H, k.shape[1], _ptr(idx), idx.shape[2], _ptr(counts),
                                           float(sm_scale), _ptr(mask), mask.stride(0), mask.shape[1], 1 if mask_by_slot else 0,
                                           _ptr(out), _ptr(ws), ws.numel(), _stream(q)), "ha_sparse_decode_masked")
        return
    _check(lib.ha_sparse_decode(*_kv_args(q, k, v), B, H, k.shape[1], _ptr(idx), idx.shape[2], _ptr(counts),
                                float(sm_scale), _ptr(out), _ptr(ws), ws.numel(), _stream(q)), "ha_sparse_decode")


def window_partial(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
                   init_budget: int, recent_budget: int, sm_scale: float, win: torch.Tensor) -> None:
    """Attention over the sink and recent windows only -> win [B, H, 130] fp32 (acc[128], m, l), unnormalised."""
    _require_cuda(q, k, v, seq_lens, win)
    lib = load_library()
    B, H, _ = q.shape
    assert win.dtype == torch.float32 and win.is_contiguous() and win.numel() == B * H * 130
    _check(lib.ha_window_partial(*_kv_args(q, k, v), B, H, k.shape[1], max_seq_len, _ptr(seq_lens), init_budget, recent_budget,
                                 float(sm_scale), _ptr(win), _stream(q)), "ha_window_partial")


def sparse_decode_heavy(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor, counts: torch.Tensor,
                        sm_scale: float, out: torch.Tensor, ws: torch.Tensor, win: torch.Tensor, init_budget: int,
                        recent_budget: int, max_seq_len: int, seq_lens: Optional[torch.Tensor]) -> None:
    """`sparse_decode` that skips the window entries of the lists and merges the partial made by `window_partial`."""
    _require_cuda(q, k, v, idx, counts, out, ws, win, seq_lens)
    lib = load_library()
    B, H, _ = q.shape
    assert out.is_contiguous() and out.dtype == q.dtype and idx.is_contiguous() and counts.is_contiguous()
    _check(lib.ha_sparse_decode_heavy(*_kv_args(q, k, v), B, H, k.shape[1], _ptr(idx), idx.shape[2], _ptr(counts),
                                      float(sm_scale), _ptr(out), _ptr(ws), ws.numel(), _ptr(win), init_budget, recent_budget,
                                      max_seq_len, _ptr(seq_lens), _stream(q)), "ha_sparse_decode_heavy")


def dense_decode_workspace_bytes(B, H, max_seq_len) -> int:
    return load_library().ha_dense_decode_workspace_bytes(B, H, max_seq_len)


def dense_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, max_seq_len: int, seq_lens: Optional[torch.Tensor],
                 sm_scale: float, out: torch.Tensor, ws: torch.Tensor) -> None:
    _require_cuda(q, k, v, seq_lens, out, ws)
    lib = load_library()
    B, H, _ = q.shape
    assert out.is_contiguous() and out.dtype == q.dtype
    _check(lib.ha_dense_decode(*_kv_args(q, k, v), B, H, k.shape[1], max_seq_len, _ptr(seq_lens), float(sm_scale),
                               _ptr(out), _ptr(ws), ws.numel(), _stream(q)), "ha_dense_decode")


# ------------------------------------------------------------------------------------------ decoder plumbing
def rope_append(qkv: torch.Tensor, n_q_heads: int, n_kv_heads: int, pos: int, inv_freq: torch.Tensor, q_out: torch.Tensor,
                k_cache: torch.Tensor, v_cache: torch.Tensor, pos_dev: Optional[torch.Tensor] = None) -> None:
    """qkv [B, (H + 2 Hkv) * 128] of one new token per sequence -> rotated q into q_out [B, H, 128], rotated k and v into
    the caches [B, Hkv, S_cap, 128] at position pos (or pos_dev[b])."""
    _require_cuda(qkv, inv_freq, q_out, k_cache, v_cache, pos_dev)
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and q_out.is_contiguous() and q_out.dtype == qkv.dtype == k_cache.dtype == v_cache.dtype
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() == 64 and inv_freq.is_contiguous()
    assert k_cache.stride() == v_cache.stride() and k_cache.stride(3) == 1
    B = qkv.shape[0]
    _check(load_library().ha_rope_append(_ptr(qkv), qkv.stride(0), _DTYPE[qkv.dtype], B, n_q_heads, n_kv_heads, int(pos), _ptr(pos_dev),
                                         _ptr(inv_freq), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0),
                                         k_cache.stride(1), k_cache.stride(2), k_cache.shape[2], _stream(qkv)), "ha_rope_append")


def rope_encode_step(qkv: torch.Tensor, n_q_heads: int, n_kv_heads: int, pos: int, inv_freq: torch.Tensor, q_out: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, wk: torch.Tensor, wq: torch.Tensor, n_layers: int, int_dim: int,
                     final_dim: int, kcodes: torch.Tensor, qcodes: torch.Tensor, pos_dev: Optional[torch.Tensor] = None,
                     arith: int = HA_ARITH_F32) -> None:
    """`rope_append` and `encode_step` of a decode step in one launch: the rows of qkv [B, (H + 2 Hkv) * 128] are rotated,
    written to q_out / the caches at position pos (or pos_dev[b]), and what was written is hashed into kcodes (at the same
    position) and qcodes."""
    _require_cuda(qkv, inv_freq, q_out, k_cache, v_cache, wk, wq, kcodes, qcodes, pos_dev)
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and q_out.is_contiguous() and q_out.dtype == qkv.dtype == k_cache.dtype == v_cache.dtype
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() == 64 and inv_freq.is_contiguous()
    assert k_cache.stride() == v_cache.stride() and k_cache.stride(3) == 1
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == kcodes.shape[3] and qcodes.is_contiguous()
    B = qkv.shape[0]
    assert kcodes.dtype == torch.int32 and qcodes.dtype == torch.int32 and qcodes.numel() == B * n_q_heads * (final_dim // 32)
    assert pos_dev is not None or int(pos) < kcodes.shape[2]
    _check(load_library().ha_rope_encode_step(
        _ptr(qkv), qkv.stride(0), _DTYPE[qkv.dtype], B, n_q_heads, n_kv_heads, wk.shape[0], int(pos), _ptr(pos_dev), _ptr(inv_freq),
        _ptr(q_out), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), k_cache.shape[2],
        _ptr(wk), _ptr(wq), n_layers, 128, int_dim, final_dim, arith, _ptr(kcodes), kcodes.stride(0), kcodes.stride(1), _ptr(qcodes),
        _stream(qkv)), "ha_rope_encode_step")


def rope_encode_step_cos_sin(qkv: torch.Tensor, n_q_heads: int, n_kv_heads: int, pos: int, cos: torch.Tensor, sin: torch.Tensor,
                             q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, wk: torch.Tensor, wq: torch.Tensor,
                             n_layers: int, int_dim: int, final_dim: int, kcodes: torch.Tensor, qcodes: torch.Tensor,
                             arith: int = HA_ARITH_F32) -> None:
    """`rope_encode_step` with the rotation given as the cos / sin rows a transformers layer receives: [B or 1, 128] of the
    dtype of qkv (any leading singleton dimensions squeezed by the caller).  k_cache / v_cache [B, Hkv, capacity, 128]: the
    new key and value go to token position `pos`."""
    _require_cuda(qkv, cos, sin, q_out, k_cache, v_cache, wk, wq, kcodes, qcodes)
    B = qkv.shape[0]
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and q_out.is_contiguous() and q_out.dtype == qkv.dtype == k_cache.dtype == v_cache.dtype
    assert cos.dtype == sin.dtype == qkv.dtype and cos.dim() == 2 and cos.shape == sin.shape and cos.shape[1] == 128
    assert cos.shape[0] in (1, B) and cos.stride(1) == 1 and sin.stride() == cos.stride()
    assert k_cache.stride() == v_cache.stride() and k_cache.stride(3) == 1
    assert kcodes.stride(3) == 1 and kcodes.stride(2) == kcodes.shape[3] and qcodes.is_contiguous()
    assert kcodes.dtype == torch.int32 and qcodes.dtype == torch.int32 and qcodes.numel() == B * n_q_heads * (final_dim // 32)
    assert 0 <= int(pos) < kcodes.shape[2] and int(pos) < k_cache.shape[2]
    _check(load_library().ha_rope_encode_step_cos_sin(
        _ptr(qkv), qkv.stride(0), _DTYPE[qkv.dtype], B, n_q_heads, n_kv_heads, wk.shape[0], int(pos), None, _ptr(cos), _ptr(sin),
        0 if cos.shape[0] == 1 else cos.stride(0), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), k_cache.stride(1),
        k_cache.stride(2), k_cache.shape[2], _ptr(wk), _ptr(wq), n_layers, 128, int_dim, final_dim, arith, _ptr(kcodes), kcodes.stride(0),
        kcodes.stride(1), _ptr(qcodes), _stream(qkv)), "ha_rope_encode_step_cos_sin")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """gate_up [B, 2F] (gate | up) -> out [B, F] = silu(gate) * up."""
    _require_cuda(gate_up, out)
    assert gate_up.dim() == 2 and gate_up.stride(1) == 1 and out.is_contiguous() and out.dtype == gate_up.dtype
    B, F = out.shape
    _check(load_library().ha_swiglu(_ptr(gate_up), gate_up.stride(0), _DTYPE[gate_up.dtype], B, F, _ptr(out), _stream(gate_up)), "ha_swiglu")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """x [M, K] -> out [M, K] = round(round(x * rsqrt(mean x^2 + eps)) * weight): the two roundings of LlamaRMSNorm."""
    _require_cuda(x, weight, out)
    assert x.dim() == 2 and out.shape == x.shape and x.stride(1) == 1 and out.stride(1) == 1 and weight.is_contiguous()
    assert weight.dtype == x.dtype == out.dtype and weight.numel() == x.shape[1]
    _check(load_library().ha_rmsnorm(_ptr(x), x.stride(0), _ptr(weight), _DTYPE[x.dtype], x.shape[0], x.shape[1], float(eps), _ptr(out),
                                     out.stride(0), _stream(x)), "ha_rmsnorm")


HA_ACT_NONE, HA_ACT_SWIGLU = 0, 1


LINEAR_SKINNY_MAX_ROWS = 16     # rows of x that ha_linear_skinny takes
LINEAR_TILED_MAX_K = 8192       # inputs that ha_linear_tiled takes for up to 16 rows of x
LINEAR_TILED_MAX_ROWS = 32      # rows of x that ha_linear_tiled takes (above 16: up to LINEAR_TILED_MAX_K / 2 inputs)


def linear_tiled_applies(rows: int, k: int) -> bool:
    return rows <= 16 and k <= LINEAR_TILED_MAX_K or rows <= LINEAR_TILED_MAX_ROWS and k <= LINEAR_TILED_MAX_K // 2


def pack_weight_tiles(w: torch.Tensor, glu: bool = False) -> torch.Tensor:
    """The tiled copy of w [N, K] bf16 that `linear_tiled` reads (glu: w = [gate rows; up rows], tiles of 8 + 8)."""
    _require_cuda(w)
    assert w.dim() == 2 and w.dtype == torch.bfloat16 and w.stride(1) == 1
    N, K = w.shape
    n = load_library().ha_weight_tiles_elems(N, K, 1 if glu else 0)
    if n <= 0:
        raise ValueError(f"a [{N}, {K}] matrix cannot be tiled (K a multiple of 32, an even N for gate/up)")
    tiles = torch.empty(n, dtype=torch.bfloat16, device=w.device)
    _check(load_library().ha_pack_weight_tiles(_ptr(w), w.stride(0), N, K, 1 if glu else 0, _ptr(tiles), _stream(w)), "ha_pack_weight_tiles")
    return tiles


def linear_tiled(x: torch.Tensor, tiles: torch.Tensor, N: int, out: torch.Tensor, residual: Optional[torch.Tensor] = None,
                 swiglu: bool = False) -> torch.Tensor:
    """out [M, N] (or [M, N / 2] with swiglu) = x [M, K] . W^T (+ residual) from the tiled copy of W [N, K].  M <= 16 (no
    activation when K > 8192), or M <= 32 with K <= 4096."""
    _require_cuda(x, tiles, out, residual)
    assert x.dim() == 2 and x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and x.stride(1) == 1 and out.stride(1) == 1
    M, K = x.shape
    assert tiles.dtype == torch.bfloat16 and tiles.is_contiguous()
    assert tiles.numel() == load_library().ha_weight_tiles_elems(N, K, 1 if swiglu else 0), "tiles of another shape"
    assert out.shape == (M, N // 2 if swiglu else N)
    assert residual is None or (residual.shape == (M, N) and residual.dtype == torch.bfloat16 and residual.stride(1) == 1)
    _linear_tiled_unchecked(x, tiles, N, out, residual, swiglu)
    return out


def _linear_tiled_unchecked(x, tiles, N, out, residual=None, swiglu=False):
    _check(load_library().ha_linear_tiled(x.data_ptr(), x.stride(0), tiles.data_ptr(), _ptr(residual),
                                          residual.stride(0) if residual is not None else 0,
                                          HA_ACT_SWIGLU if swiglu else HA_ACT_NONE, out.data_ptr(), out.stride(0), x.shape[0], N,
                                          x.shape[1], _stream(x)), "ha_linear_tiled")


def _linear_skinny_unchecked(x, w, out, residual=None, norm_weight=None, eps=0.0, swiglu=False):
    """`linear_skinny` for callers that made these tensors themselves (2-D bf16 on one GPU, rows contiguous): no checks on
    the Python side - a decode layer's seven launches should not cost the host more than they cost the GPU.  The library
    still validates sizes, strides and alignment."""
    lib = _lib or load_library()
    M, K = x.shape
    N = w.shape[0]
    if norm_weight is None and not swiglu:
        st = lib.ha_linear_skinny(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None if residual is None else residual.data_ptr(),
                                  0 if residual is None else residual.stride(0), out.data_ptr(), out.stride(0), M, N, K, _stream(x))
    else:
        st = lib.ha_linear_skinny_fused(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None if residual is None else residual.data_ptr(),
                                        0 if residual is None else residual.stride(0), None if norm_weight is None else norm_weight.data_ptr(),
                                        eps, HA_ACT_SWIGLU if swiglu else HA_ACT_NONE, out.data_ptr(), out.stride(0), M, N, K, _stream(x))
    if st:
        _check(st, "ha_linear_skinny")
    return out


def linear_skinny(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, residual: Optional[torch.Tensor] = None,
                  norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-5, swiglu: bool = False) -> torch.Tensor:
    """out [M, N] = x [M, K] @ w[N, K]^T (+ residual [M, N]); bf16, M <= 16.  Streams w once.
    norm_weight [K]: x is RMS-normalised first (M <= 8, K <= 16384).  swiglu: w = [gate rows; up rows], out [M, N / 2] =
    silu(gate) * up (M <= 8, K <= 16384, no residual)."""
    _require_cuda(x, w, out, residual, norm_weight)
    assert x.dtype == w.dtype == out.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2 and out.dim() == 2
    assert x.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1 and (residual is None or (residual.stride(1) == 1 and residual.dtype == x.dtype))
    M, K = x.shape
    N = w.shape[0]
    n_out = N // 2 if swiglu else N
    assert w.shape[1] == K and out.shape == (M, n_out) and (residual is None or residual.shape == (M, N))
    res_stride = residual.stride(0) if residual is not None else 0
    if norm_weight is None and not swiglu:
        _check(load_library().ha_linear_skinny(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), res_stride, _ptr(out),
                                               out.stride(0), M, N, K, _stream(x)), "ha_linear_skinny")
        return out
    assert norm_weight is None or (norm_weight.dtype == torch.bfloat16 and norm_weight.shape == (K,) and norm_weight.is_contiguous())
    _check(load_library().ha_linear_skinny_fused(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), res_stride, _ptr(norm_weight),
                                                 float(eps), HA_ACT_SWIGLU if swiglu else HA_ACT_NONE, _ptr(out), out.stride(0), M, N, K,
                                                 _stream(x)), "ha_linear_skinny_fused")
    return out
