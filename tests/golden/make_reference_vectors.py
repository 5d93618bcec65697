"""One-off generator of golden vectors from the reference's own code (run in the build container only).

It imports /root/reference/hashattention/hashattention_llama.py on the CPU and records, for small seeded
inputs, what `USA.forward(hard=True)` and `LlamaAttention_heavy_hitter.compute_mask_multi` return.  These
two functions fix conventions that no test of the reference pins (which K MLP reads which repeated KV head,
the exact extent of the sink / recent windows for every query row, budget truncation, threshold mode), so
their outputs are committed as data: tests/golden/reference_vectors.npz.

    python tests/golden/make_reference_vectors.py

The reference sorts without `stable=True`; the masks stored here are its raw output, to be compared up to
the choice among equal scores (oracle.tie_invariant_equal), never bit for bit.
"""
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")


def main():
    sys.dont_write_bytecode = True      # the reference tree is read-only: no __pycache__ beside its sources
    sys.path.insert(0, REF)
    from hashattention import hashattention_llama as ref   # prints "CENTER 0"

    torch.manual_seed(1234)
    H, Hkv, d, S = 4, 2, 128, 64
    cfg = {"lth_int_dim": 32, "lth_final_dim": 32, "lth_thold": 0, "lth_num_layers": 3}
    usa = ref.USA(H, d, cfg)
    out = {}
    # weights, flattened in state-dict order
    sd = usa.state_dict()
    out["state_keys"] = np.array(list(sd.keys()))
    for i, (k, v) in enumerate(sd.items()):
        out[f"w{i}"] = v.numpy()

    K = torch.randn(2, Hkv, S, d)
    out["K"] = K.numpy()
    Krep = ref.repeat_kv(K, H // Hkv)
    for name, q_len in (("q1", 1), ("q5", 5)):
        Q = torch.randn(2, H, q_len, d)
        out[f"{name}_Q"] = Q.numpy()
        span, ksign = usa(Krep, Q, hard=True)
        out[f"{name}_span"] = span.detach().numpy()
        out[f"{name}_ksign"] = ksign.detach().numpy().astype(np.int8)
        for tag, init, recent, heavy, mode, depth in (("a", 4, 6, 0.25, "simple", 0), ("b", 0, 3, 10.0, "simple", 0),
                                                      ("c", 8, 8, 0.125, "thold", 2), ("d", 50, 60, 0.5, "simple", 0)):
            ns = types.SimpleNamespace(usa_module=usa, usa_module_dtype=torch.float32, past_key_signatures=None,
                                       recent_budget=recent, init_budget=init, heavy_budget=heavy, usa_eval_mode=mode,
                                       usa_retrieve_depth=depth, num_heads=H)
            mask = ref.LlamaAttention_heavy_hitter.compute_mask_multi(ns, Krep, Q)
            out[f"{name}_{tag}_mask"] = np.packbits(mask.numpy(), axis=-1)
            out[f"{name}_{tag}_params"] = np.array([init, recent, heavy, 0 if mode == "simple" else 1, depth], dtype=np.float64)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
