"""The decoder-step harness (RMSNorm, fused QKV, rotate-half RoPE, in-place cache append, sparse attention,
SwiGLU, lm_head) against a `transformers` Llama of the same weights whose attention layers were converted with
`convert_usa`: both run the HIP attention, so this checks the plumbing around it.  fp32, tight tolerance."""
import pytest
import torch
from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM

from hashattention import hashattention_llama as hl
from hashattention.decoder import LlamaShapedDecoder
from hashattention.synthetic import UsaWeights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _linears(seqs):
    return [[(m.weight.detach().float().cpu(), m.bias.detach().float().cpu()) for m in seq if isinstance(m, torch.nn.Linear)]
            for seq in seqs]


def test_decoder_step_matches_converted_llama():
    print("\n[case] decoder step vs converted Llama", flush=True)
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, vocab_size=512, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5)
    usa_cfg = dict(lth_init_dim=128, lth_final_dim=32, lth_thold=0, lth_num_layers=3, init_budget=8, heavy_budget=0.125,
                   recent_budget=8, usa_retrieve_depth=6, usa_eval_mode="simple")
    for k, v in usa_cfg.items():
        setattr(cfg, k, v)
    model = LlamaForCausalLM(cfg).bfloat16().float()
    usa = hl.load_usa(cfg, None)
    model = hl.convert_usa(model.to(DEV), cfg, usa, collect_stats=False, train_usa=False).float()

    B, S0, steps = 2, 300, 3
    ids = torch.randint(0, cfg.vocab_size, (B, S0 + steps), generator=torch.Generator().manual_seed(1)).to(DEV)
    cache = DynamicCache()
    want = []
    with torch.no_grad():
        model(ids[:, :S0], past_key_values=cache, use_cache=True)        # q_len > 128: dense prefill
        keys = [cache.layers[l].keys.clone() for l in range(2)]
        values = [cache.layers[l].values.clone() for l in range(2)]
        for t in range(steps):
            want.append(model(ids[:, S0 + t:S0 + t + 1], past_key_values=cache, use_cache=True).logits[:, 0].float().cpu())

    dec = LlamaShapedDecoder(n_layers=2, hidden=512, ffn=1024, n_heads=4, n_kv_heads=2, head_dim=128, vocab=512,
                             rope_theta=500000.0, rms_eps=1e-5, n_code_heads=4, lth_num_layers=3, lth_int_dim=128,
                             lth_final_dim=32, init_budget=8, recent_budget=8, heavy_budget=0.125, dtype=torch.float32, device=DEV)
    dec.load_hf_llama(model)
    weights = [UsaWeights(k=_linears(u.learning_to_hash_transformation_k), q=_linears(u.learning_to_hash_transformation_q))
               for u in usa]
    dec.allocate(B, 512, weights)
    dec.load_cache(keys, values)
    with torch.no_grad():
        for t in range(steps):
            got = dec.decode_step(ids[:, S0 + t]).float().cpu()
            err = (got - want[t]).abs().max().item()
            print(f"step {t}: max-abs logit difference {err:.2e}", flush=True)
            assert err < 2e-3, err
    assert dec.seq_len == S0 + steps
