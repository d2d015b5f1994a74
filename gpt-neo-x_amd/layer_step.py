"""Time one transformer layer (forward + backward) built from the fused kernels, on one GPU.

    python gpt-neo-x_amd/layer_step.py [--config pythia-1.4b|llama2-7b|mistral-7b] [--steps 20] [--warmup 5] [--dropout 0.0]

Prints one JSON line with the time per step. Under ``rocprofv3 --kernel-trace --stats`` the kernel table shows how
the step divides between the library GEMMs and the kernels of libneox_hotpath.so (names starting with ``nhp::``).
Synthetic input, random parameters.
"""
import argparse
import json
import os
import sys
import time
import types

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

CONFIGS = {
    # hidden, heads, sequence, batch, then what differs between the two families
    "pythia-1.4b": dict(hidden_size=2048, num_attention_heads=16, seq_length=2048, batch=8, norm="layernorm",
                        activation="gelu", rotary_pct=0.25, gpt_j_residual=True, use_bias=True, intermediate_size=None),
    "llama2-7b": dict(hidden_size=4096, num_attention_heads=32, seq_length=4096, batch=1, norm="rmsnorm",
                      activation="swiglu", rotary_pct=1.0, gpt_j_residual=False, use_bias=False, intermediate_size=11008 * 3),
    # grouped-query attention (8 key/value heads for 32 query heads) and a sliding window of 4096 keys
    "mistral-7b": dict(hidden_size=4096, num_attention_heads=32, num_kv_heads=8, seq_length=8192, batch=1, norm="rmsnorm",
                       activation="swiglu", rotary_pct=1.0, gpt_j_residual=False, use_bias=False,
                       intermediate_size=14336 * 3, sliding_window_width=4096),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="pythia-1.4b", choices=sorted(CONFIGS))
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--dropout", type=float, default=0.0)
    a = ap.parse_args()

    import torch

    from megatron.model.transformer_layer import TransformerLayer

    if not torch.cuda.is_available():
        raise SystemExit("layer_step.py needs a GPU")
    c = CONFIGS[a.config]
    cfg = types.SimpleNamespace(
        hidden_size=c["hidden_size"], num_attention_heads=c["num_attention_heads"], seq_length=c["seq_length"],
        precision="bfloat16", pos_emb="rotary", rotary_pct=c["rotary_pct"], rotary_emb_base=10000, rope_fusion=True,
        norm=c["norm"], layernorm_epsilon=1e-5, rms_norm_epsilon=1e-6, layernorm_fusion=False, rmsnorm_fusion=False,
        activation=c["activation"], bias_gelu_fusion=True, onnx_safe=False,
        scaled_upper_triang_masked_softmax_fusion=True, scaled_masked_softmax_fusion=False,
        attention_softmax_in_fp32=True, apply_query_key_layer_scaling=False, attention_dropout=a.dropout,
        hidden_dropout=a.dropout, bias_dropout_fusion=True, gpt_j_residual=c["gpt_j_residual"], gpt_j_tied=False,
        use_bias_in_mlp=c["use_bias"], use_bias_in_attn_linear=c["use_bias"], intermediate_size=c["intermediate_size"],
        expansion_factor=None, num_kv_heads=c.get("num_kv_heads"), sliding_window_width=c.get("sliding_window_width"))
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    def mask_func(scores, mask):
        return scores.masked_fill(mask, torch.finfo(scores.dtype).min)

    layer = TransformerLayer(cfg, mask_func, layer_number=1, rotary=True).to(dev).to(torch.bfloat16).train()
    s, b, h = c["seq_length"], c["batch"], c["hidden_size"]
    x = torch.randn((s, b, h), device=dev).to(torch.bfloat16).requires_grad_(True)
    g = torch.randn((s, b, h), device=dev).to(torch.bfloat16)
    pos = torch.arange(s, device=dev)
    mask = (pos.view(1, s) > pos.view(s, 1)).view(1, 1, s, s)

    def step():
        layer.zero_grad(set_to_none=True)
        x.grad = None
        layer(x, mask).backward(g)

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.steps
    print(json.dumps({"workload": "transformer layer forward + backward", "config": a.config, "tokens": s * b,
                      "hidden_size": h, "dropout": a.dropout, "steps": a.steps, "warmup": a.warmup,
                      "ms_per_step": round(ms, 3)}), flush=True)


if __name__ == "__main__":
    main()
