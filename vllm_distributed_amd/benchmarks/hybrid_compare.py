"""Prefill and decode throughput of a Nositar, Rapovik, Sevazen or Lefolorn stack beside the closest existing models of
equal size, random weights.

    python bench.py --compare-nositar [--sizes small,medium] [--batch 32] [--input-len 2048] [--output-len 64]
    python bench.py --compare-rapovik [...]        (rapovik beside jamba-moe)
    python bench.py --compare-sevazen [...]        (sevazen beside mixtral-swa)
    python bench.py --compare-lefolorn [...]       (lefolorn beside sevazen and mixtral-swa)

Per size three engines run one after the other, each in a process of its own (``--one`` is the child's entry):
  nositar      alternating sigmoid head-mixing attention (window + kept first tokens) and gated delta-rule layers,
               two residual streams, ReLU-gated feed-forward
  llama-swa    a Llama stack of the same width, depth, heads and feed-forward with the same sliding window (the
               framework's softmax attention kernels)
  jamba        the framework's attention + recurrent (Mamba) hybrid of the same width, depth and feed-forward
  jamba-moe    the same with 8 routed experts (two per token) in every other layer
  rapovik      latent window attention, Mamba-2 and mLSTM mixers in turn over an fp32 residual with norms around every
               sub-layer; clamped gated feed-forwards, dense and routed (8 experts, two per token, one shared) in turn
  sevazen      window attention with sinks and a short convolution and differential attention inside chunks in turn,
               fp32 residual with layer norms on the sub-layers' outputs, 8 routed squared-ReLU experts (two per token)
               plus a shared expert in every layer
  lefolorn     latent attention with sinks, distance-bias attention with an output gate and soft-capped window attention
               in turn; both sub-layers of a layer read one group norm of the fp32 residual and join it behind layer
               scales and per-channel sigmoid gates; every layer has 8 routed gated experts and 2 identity outputs (two
               choices per token, from the better of two groups) plus a shared expert
  mixtral-swa  a Mixtral stack of the same width, depth and heads with the same sliding window and 8 routed gated
               experts (two per token) of equal weight count
Prefill: ``batch`` prompts of ``input-len`` tokens, one generated token.  Decode: the same requests generating
``output-len`` tokens, the prefill time taken off.  One JSON line per (size, model).
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import tempfile
import time

SIZES = {
    # width, layers, heads, kv heads, head dim, feed-forward, window, vocab
    "small": dict(width=1024, layers=8, heads=16, kv_heads=4, dim=64, ff=4096, window=512, vocab=32000),
    "medium": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=8192, window=1024, vocab=32000),
    "large": dict(width=4096, layers=4, heads=32, kv_heads=8, dim=128, ff=14336, window=1024, vocab=32000),
}


def nositar_config(s: dict) -> dict:
    att = {"type": "attention", "mlp": {"kind": "dense", "ff": s["ff"]},
           "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"],
                     "scale": s["dim"] ** -0.5, "mask": {"size": s["window"], "keep_first": 4}}}
    dh = max(s["width"] // 128, 1)
    delta = {"type": "channel_delta", "mlp": {"kind": "dense", "ff": s["ff"]},
             "mixer": {"heads": dh, "kv_heads": dh, "dim": 128, "vdim": 128, "conv": 4, "decay_rank": 64,
                       "gate_rank": 64}}
    return {"architecture": "Nositar", "vocab": s["vocab"], "width": s["width"], "streams": 2, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "logit_softcap": 30.0,
            "layers": [att if i % 2 == 0 else delta for i in range(s["layers"])]}


def llama_config(s: dict) -> dict:
    return {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_size": s["width"],
            "intermediate_size": s["ff"], "num_hidden_layers": s["layers"], "num_attention_heads": s["heads"],
            "num_key_value_heads": s["kv_heads"], "head_dim": s["dim"], "vocab_size": s["vocab"],
            "sliding_window": s["window"], "max_position_embeddings": 32768, "rms_norm_eps": 1e-6,
            "rope_theta": 10000.0, "tie_word_embeddings": False, "torch_dtype": "bfloat16"}


def jamba_config(s: dict) -> dict:
    return {"architectures": ["JambaForCausalLM"], "model_type": "jamba", "hidden_size": s["width"],
            "intermediate_size": s["ff"], "num_hidden_layers": s["layers"], "num_attention_heads": s["heads"],
            "num_key_value_heads": s["kv_heads"], "vocab_size": s["vocab"], "attn_layer_period": 2,
            "attn_layer_offset": 0, "expert_layer_period": 2, "expert_layer_offset": 1, "num_experts": 1,
            "num_experts_per_tok": 1, "mamba_expand": 2, "mamba_d_state": 16, "mamba_d_conv": 4,
            "mamba_dt_rank": max(s["width"] // 16, 1), "mamba_proj_bias": False, "mamba_conv_bias": True,
            "rms_norm_eps": 1e-6, "max_position_embeddings": 32768, "tie_word_embeddings": False,
            "torch_dtype": "bfloat16"}


def jamba_moe_config(s: dict) -> dict:
    """Jamba with routed experts (8, two per token) in every other layer, as the checkpoints of that family have."""
    return dict(jamba_config(s), num_experts=8, num_experts_per_tok=2)


def rapovik_config(s: dict) -> dict:
    """Per four layers: latent window attention, Mamba-2, mLSTM, Mamba-2; dense feed-forwards alternate with routed
    experts (8, two per token from the better of two groups, plus a shared expert of a quarter of the width)."""
    w, ff = s["width"], s["ff"]
    rank, rot = (128, 32) if w <= 1024 else (512, 64)
    dense = {"kind": "dense", "ff": ff, "limit": 7.0}
    moe = {"kind": "moe", "router": {"experts": 8, "top": 2, "groups": {"count": 2, "keep": 1}},
           "expert": {"ff": ff, "limit": 7.0}, "shared": {"ff": ff // 4, "limit": 7.0}}
    att = {"type": "latent_attention",
           "mixer": {"heads": s["heads"], "dim": s["dim"], "rot_dim": rot, "vdim": s["dim"], "kv_rank": rank,
                     "scale": (s["dim"] + rot) ** -0.5, "mask": {"size": s["window"]},
                     "rot": {"base": 10000.0, "dims": rot}}}
    mamba = {"type": "mamba2", "mixer": {"heads": 2 * w // 64, "vdim": 64, "state": 64, "groups": 1, "conv": 4,
                                         "norm_groups": 1}}
    mh = max(w // 128, 1)
    mlstm = {"type": "mlstm", "mixer": {"heads": mh, "dim": 64, "vdim": 2 * w // mh, "gate_cap": 15.0}}
    cycle = [att, mamba, mlstm, mamba]
    return {"architecture": "Rapovik", "vocab": s["vocab"], "width": w, "norm": {"eps": 1e-6},
            "layers": [dict(cycle[i % 4], mlp=dense if i % 2 == 0 else moe) for i in range(s["layers"])]}


def mixtral_swa_config(s: dict) -> dict:
    """A Mixtral stack with a sliding window: softmax attention + 8 routed gated experts (two per token) per layer."""
    return {"architectures": ["MixtralForCausalLM"], "model_type": "mixtral", "hidden_size": s["width"],
            "intermediate_size": s["ff"], "num_hidden_layers": s["layers"], "num_attention_heads": s["heads"],
            "num_key_value_heads": s["kv_heads"], "head_dim": s["dim"], "vocab_size": s["vocab"],
            "num_local_experts": 8, "num_experts_per_tok": 2, "sliding_window": s["window"],
            "max_position_embeddings": 32768, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
            "tie_word_embeddings": False, "torch_dtype": "bfloat16"}


def sevazen_config(s: dict) -> dict:
    """Window attention (sink, 4-tap convolution, half of each head rotated) and differential attention inside chunks of
    the window's size (half as many heads: two score maps each) in turn; every layer has 8 routed squared-ReLU experts
    (two per token; 1.5 x the width of the gated experts beside them, for equal weights) and a shared expert."""
    w, ff, d = s["width"], s["ff"], s["dim"]
    moe = {"kind": "moe", "router": {"experts": 8, "top": 2}, "expert": {"ff": ff * 3 // 2}, "shared": {"ff": ff // 4}}
    win = {"type": "attention",
           "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": d, "vdim": d, "scale": d ** -0.5, "conv": 4,
                     "mask": {"size": s["window"]},
                     "rot": {"base": 500000.0, "dims": d // 2,
                             "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}}
    dif = {"type": "attention_2",
           "mixer": {"heads": s["heads"] // 2, "kv_heads": max(s["kv_heads"] // 2, 1), "dim": d, "vdim": d,
                     "scale": d ** -0.5, "diff": 0.5, "mask": {"size": s["window"]},
                     "rot": {"base": 10000.0, "dims": d // 2,
                             "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}}
    return {"architecture": "Sevazen", "vocab": s["vocab"], "width": w, "norm": {"eps": 1e-6},
            "layers": [dict(win if i % 2 == 0 else dif, mlp=moe) for i in range(s["layers"])]}


def lefolorn_config(s: dict) -> dict:
    """Latent attention (sinks; latent of 128 + 32 for heads of 64, 512 + 64 for heads of 128: the sizes the
    matrix-core latent kernel has), distance-bias attention (32 buckets up to half the window, query temperature, output
    gate, one more 1 in the denominator) and soft-capped window attention (half of each head rotated) in turn, values
    mixed across the last two kinds; gated experts of the Mixtral stack's width, 8 + 2 identity outputs in two groups of
    which the better one is kept, two choices per token, a shared expert of a quarter of the width."""
    w, ff, d = s["width"], s["ff"], s["dim"]
    moe = {"kind": "moe", "router": {"experts": 8, "identity": 2, "top": 2, "groups": {"count": 2, "keep": 1}},
           "expert": {"ff": ff}, "shared": {"ff": ff // 4}}
    rank, rot = (128, 32) if d <= 64 else (512, 64)
    lat = {"type": "latent_attention",
           "mixer": {"heads": s["heads"], "dim": d, "rot_dim": rot, "vdim": d, "kv_rank": rank, "q_rank": w // 2,
                     "scale": (d + rot) ** -0.5, "rot": {"base": 10000.0, "dims": rot}}}
    common = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": d, "vdim": d, "scale": d ** -0.5, "v_mix": True}
    bias = {"type": "attention", "mixer": dict(common, bias_max=s["window"] // 2, bias_rows=32,
                                               q_temp={"coef": 0.25, "every": 512})}
    cap = {"type": "attention_2", "mixer": dict(common, mask={"size": s["window"]}, softcap=30.0,
                                                rot={"base": 10000.0, "dims": d // 2})}
    return {"architecture": "Lefolorn", "vocab": s["vocab"], "width": w, "norm": {"eps": 1e-6, "groups": 8},
            "layers": [dict((lat, bias, cap)[i % 3], mlp=moe) for i in range(s["layers"])]}


MODELS = {"lefolorn": lefolorn_config, "sevazen": sevazen_config, "mixtral-swa": mixtral_swa_config, "nositar": nositar_config, "llama-swa": llama_config, "jamba": jamba_config, "jamba-moe": jamba_moe_config,
          "rapovik": rapovik_config}


def run_one(kind: str, size: str, batch: int, input_len: int, output_len: int, eager: bool) -> dict:
    import torch
    from vllm_distributed_amd import LLM, SamplingParams
    folder = tempfile.mkdtemp(prefix=f"vda_cmp_{kind}_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(MODELS[kind](SIZES[size]), f)
    llm = LLM(model=folder, load_format="dummy", skip_tokenizer_init=True, dtype="bfloat16",
              max_model_len=input_len + output_len + 16, max_num_seqs=max(batch, 8),
              max_num_batched_tokens=16384, enable_prefix_caching=False, gpu_memory_utilization=0.6,
              enforce_eager=eager, seed=0)
    vocab = SIZES[size]["vocab"]

    def prompts(seed):
        g = torch.Generator().manual_seed(seed)
        return torch.randint(10, vocab - 10, (batch, input_len), generator=g).tolist()

    def timed(seed, new_tokens):
        sp = SamplingParams(temperature=0.0, max_tokens=new_tokens, ignore_eos=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        llm.generate(prompt_token_ids=prompts(seed), sampling_params=sp)
        torch.cuda.synchronize()
        return time.perf_counter() - t0
    timed(1, 2)                                    # warm-up: allocations, library heuristics
    t_pre = min(timed(2, 1), timed(3, 1))
    t_all = min(timed(4, output_len), timed(5, output_len))
    llm.shutdown()
    t_dec = max(t_all - t_pre, 1e-9)
    return {"model": kind, "size": size, **{k: SIZES[size][k] for k in ("width", "layers", "heads", "dim", "window")},
            "batch": batch, "input_len": input_len, "output_len": output_len,
            "prefill_tokens_per_s": round(batch * input_len / t_pre, 1),
            "decode_tokens_per_s": round(batch * (output_len - 1) / t_dec, 1),
            "prefill_s": round(t_pre, 4), "decode_s": round(t_dec, 4), "dtype": "bf16",
            "data": "synthetic random token prompts, random-init weights", "decode_graphs": not eager}


def main(argv=None) -> list[dict]:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--sizes", default="small,medium")
    ap.add_argument("--models", default="nositar,llama-swa,jamba")
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--input-len", type=int, default=2048)
    ap.add_argument("--output-len", type=int, default=64)
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--one", default=None, help="internal: run one (model, size) in this process")
    a = ap.parse_args(argv)
    if a.one:
        kind, size = a.one.split(":")
        print(json.dumps(run_one(kind, size, a.batch, a.input_len, a.output_len, a.enforce_eager)), flush=True)
        return []
    rows = []
    for size in a.sizes.split(","):
        for kind in a.models.split(","):
            cmd = [sys.executable, "-m", "vllm_distributed_amd.benchmarks.hybrid_compare", "--one", f"{kind}:{size}",
                   "--batch", str(a.batch), "--input-len", str(a.input_len), "--output-len", str(a.output_len)]
            if a.enforce_eager:
                cmd.append("--enforce-eager")
            print(f"[compare] {kind} {size} ...", file=sys.stderr, flush=True)
            r = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=900)
            line = next((ln for ln in reversed(r.stdout.splitlines()) if ln.startswith("{")), None)
            if r.returncode != 0 or line is None:
                row = {"model": kind, "size": size, "error": f"exit code {r.returncode}"}
            else:
                row = json.loads(line)
            rows.append(row)
            print(json.dumps(row), flush=True)
    return rows


if __name__ == "__main__":
    main()
