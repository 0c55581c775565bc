#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, at the SmolLM2-1.7B shape with
random weights and uniform random token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--batch B] [--layers L]
                    [--prefill-tokens T] [--no-points] [--shape smollm2|llama3_8b] [--trace-only] [--decode-phases] [--portion-align A] [--mixed] [--sweep] [--kuponex] [--sepedra] [--kikarax] [--vupolix]

A step is one decode step of the whole engine (scheduler, graph replay of the model, sampling,
token hand-back) for a batch of B requests that each hold a 2,048-token context.  ``value`` is
decoded tokens per second.  One JSON line is printed; it also carries the 2,048-token prefill,
the decode step's HBM roofline, decode at batch 1 and 64 with their rooflines, the same model's true
32-bit path (decode and prefill) and, at Llama-3-8B's sizes, decode, prefill, a continuous-batching workload
of 64 requests and a trace of 128 requests with shared prefixes, cancellations and preemption whose sampled requests
are checked against solo runs.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PREFILL_TOKENS = 2048

# Layer sizes of the SmolLM2-1.7B shape: 24 layers, width 2048, 32 heads on 32 kv heads of size
# 64, feed-forward 8192, vocabulary 49152, rotary base 130000, eps 1e-5, tied embeddings.
SMOLLM2_1_7B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 49152, "hidden_size": 2048, "num_hidden_layers": 24, "num_attention_heads": 32,
    "num_key_value_heads": 32, "head_dim": 64, "intermediate_size": 8192, "rope_theta": 130000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 4096,
    "bos_token_id": 1, "eos_token_id": 2,
}
BASELINE_TOK_S = 7.26               # the reference's published SmolLM2-1.7B decode rate (one stream, 4-core CPU)


LLAMA3_8B = {
    # Llama-3-8B's sizes: 32 layers, width 4096, 32 heads on 8 kv heads of 128,
    # feed-forward 14336, vocabulary 128256, rotary base 500000 without scaling, eps 1e-5, untied head.
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
    "vocab_size": 128256, "hidden_size": 4096, "num_hidden_layers": 32, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336, "rope_theta": 500000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 8192,
    "bos_token_id": 1, "eos_token_id": 2,
}


def kuponex_shape(width: int, ff: int, groups: int, vocab: int = 32000) -> dict:
    """A Kuponex of ``groups`` x (attention over a compressed cache, matrix LSTM, two layers of gated linear attention)
    with head sizes that grow with the width as real layers' do."""
    big = width >= 4096
    heads = width // 128
    layers = []
    for _ in range(groups):
        layers.append({"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff},
                       "mixer": {"heads": heads, "dim": 128 if big else 96, "rot_dim": 64 if big else 32, "vdim": 128,
                                 "kv_rank": 512 if big else 256, "scale": (192 if big else 128) ** -0.5,
                                 "rot": {"base": 500000.0, "dims": 64 if big else 32}}})
        layers.append({"type": "mlstm", "mlp": {"kind": "dense", "ff": ff},
                       "mixer": {"heads": heads // 2, "dim": 128, "vdim": 256, "gate_cap": 15.0}})
        for _ in range(2):
            layers.append({"type": "gla", "mlp": {"kind": "dense", "ff": ff},
                           "mixer": {"heads": heads, "dim": 64, "vdim": 128, "tau": 16.0, "rank": 64}})
    return {"architecture": "Kuponex", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "layers": layers,
            "max_positions": 16384, "eos_token_id": 2}


def llama_shape(width: int, ff: int, layers: int, vocab: int = 32000) -> dict:
    """The Llama decoder of the same width, depth, feed-forward and vocabulary (heads of 128, a quarter as many kv heads)."""
    return {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "vocab_size": vocab,
            "hidden_size": width, "num_hidden_layers": layers, "num_attention_heads": width // 128,
            "num_key_value_heads": max(1, width // 512), "head_dim": 128, "intermediate_size": ff, "rope_theta": 500000.0,
            "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 16384, "bos_token_id": 1, "eos_token_id": 2}


def kuponex_comparison(bw, torch, steps: int, dtype: str, only: str = "") -> int:
    """Prefill and decode of Kuponex at two layer sizes beside the Llama decoder of equal width, depth and feed-forward:
    one JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    for name, width, ff, groups in (("2048x8192", 2048, 8192, 2), ("4096x14336", 4096, 14336, 2)):
        for arch, cfg in (("Kuponex", kuponex_shape(width, ff, groups)), ("Llama", llama_shape(width, ff, 4 * groups))):
            if only and only.lower() != arch.lower():
                continue
            model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            for tokens in (512, 2048):
                for exact in ((True, False) if arch == "Kuponex" else (True,)):
                    # (exact_cuts False: the matrix memories run a long portion in three passes over chunks)
                    m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens, exact_cuts=exact)
                    print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "prefill_tokens": tokens, "exact_cuts": exact,
                                      "ms": m["ms"], "tok_s": m["value"], "frac_of_matrix_peak": m["frac"]}), flush=True)
            for batch in (1, 8, 64):
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=2048, exact_cuts=False)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "decode_batch": batch, "context": 2048,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
            del model
            torch.cuda.empty_cache()
    return 0


def sepedra_shape(width: int, expert_ff: int, groups: int, experts: int = 32, top: int = 4, vocab: int = 32000) -> dict:
    """A Sepedra of ``groups`` x (two recurrent layers, an attention layer, an attention layer that reads the first one's
    cache), heads of 128 with a quarter as many key heads, recurrent branches as wide as the model in blocks of 128,
    feed-forwards of ``experts`` experts of which a token uses ``top``."""
    heads = width // 128
    rot = {"base": 500000.0, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    mlp = {"kind": "moe", "expert": {"ff": expert_ff, "limit": 7.0},
           "router": {"experts": experts, "top": top, "groups": {"count": 4, "keep": 2}}}
    layers = []
    for g in range(groups):
        for _ in range(2):
            layers.append({"type": "rglru", "mixer": {"width": width, "blocks": heads, "conv": 4}, "mlp": mlp})
        att = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128, "conv": 4, "scale": 128 ** -0.5, "rot": rot}
        layers.append({"type": "attention", "mixer": dict(att), "mlp": mlp})
        layers.append({"type": "attention", "mixer": dict(att, kv_from=4 * g + 2), "mlp": mlp})
    return {"architecture": "Sepedra", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "logit_softcap": 50.0,
            "layers": layers, "max_positions": 16384, "eos_token_id": 2}


def sepedra_comparison(bw, torch, steps: int, dtype: str, only: str = "") -> int:
    """Prefill and decode of Sepedra at two layer sizes beside the Llama decoder of equal width and depth whose
    feed-forward is as wide as the experts a token uses together: one JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    for name, width, expert_ff, groups in (("2048x(4x2048 of 32)", 2048, 2048, 2), ("4096x(4x3584 of 32)", 4096, 3584, 2)):
        for arch, cfg in (("Sepedra", sepedra_shape(width, expert_ff, groups)), ("Llama", llama_shape(width, 4 * expert_ff, 4 * groups))):
            if only and only.lower() != arch.lower():
                continue
            model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            for tokens in (512, 2048):
                m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "prefill_tokens": tokens,
                                  "ms": m["ms"], "tok_s": m["value"], "frac_of_matrix_peak": m["frac"]}), flush=True)
            for batch in (1, 8, 64):
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=2048)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "decode_batch": batch, "context": 2048,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
            del model
            torch.cuda.empty_cache()
    return 0


def kikarax_shape(width: int, expert_ff: int, pairs: int, experts: int = 32, top: int = 4, vocab: int = 32000) -> dict:
    """A Kikarax of ``pairs`` x (a layer with a dense feed-forward four experts wide, a layer with ``experts`` experts of
    which a token uses ``top`` beside a shared one), heads of 128 with a quarter as many key heads, chunks of 8,192
    positions, capped scores, values mixed in every layer, a table of 2^16 token pairs and learned positions."""
    heads = width // 128
    att = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "softcap": 50.0,
           "mask": {"size": 8192}, "v_mix": True}
    dense = {"kind": "dense", "ff": 4 * expert_ff, "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "scale": 2.0}, "shared": {"ff": expert_ff}}
    layers = []
    for _ in range(pairs):
        layers.append({"type": "attention", "mixer": dict(att), "mlp": dense})
        layers.append({"type": "attention", "mixer": dict(att), "mlp": moe})
    return {"architecture": "Kikarax", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "logit_scale": 0.25,
            "embedding": {"scale": 8.0, "bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 3}},
            "layers": layers, "max_positions": 16384, "eos_token_id": 2}


def kikarax_comparison(bw, torch, steps: int, dtype: str, only: str = "") -> int:
    """Prefill and decode of Kikarax at two layer sizes beside the Llama decoder of equal width and depth whose
    feed-forward is as wide as the experts a token uses together: one JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    for name, width, expert_ff, pairs in (("2048x(4x2048 of 32)", 2048, 2048, 4), ("4096x(4x3584 of 32)", 4096, 3584, 4)):
        for arch, cfg in (("Kikarax", kikarax_shape(width, expert_ff, pairs)), ("Llama", llama_shape(width, 4 * expert_ff, 2 * pairs))):
            if only and only.lower() != arch.lower():
                continue
            model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            for tokens in (512, 2048):
                m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "prefill_tokens": tokens,
                                  "ms": m["ms"], "tok_s": m["value"], "frac_of_matrix_peak": m["frac"]}), flush=True)
            for batch in (1, 8, 64):
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=2048)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "decode_batch": batch, "context": 2048,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
            del model
            torch.cuda.empty_cache()
    return 0


def vupolix_shape(width: int, expert_ff: int, experts: int = 32, top: int = 4, vocab: int = 32000) -> dict:
    """A Vupolix of six layers (time mixing and the two side-by-side mixers in turn) of which the third and fourth run
    twice: eight layer runs.  Time mixing with heads of 64, attention with heads of 128, a quarter as many key heads, half
    of each head rotated along a ramp and a window of 1,024 keys, retention with heads of 128 x 256, feed-forwards of
    ``experts`` experts in four groups of which two are kept and a token uses ``top``, beside a shared expert."""
    heads = width // 128
    mlp = {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top, "groups": {"count": 4, "keep": 2}},
           "shared": {"ff": expert_ff}}
    time_mix = {"type": "wkv", "mixer": {"heads": width // 64, "dim": 64, "rank": 64}, "mlp": mlp}
    rh = max(1, width // 256)
    both = {"type": "parallel", "mlp": mlp, "mixer": {
        "left": {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "mask": {"size": 1024},
                 "rot": {"base": 500000.0, "dims": 64, "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}},
        "right": {"heads": rh, "dim": 128, "vdim": 256, "decay": [1.0 - 2.0 ** (-5 - 3 * i / max(rh - 1, 1)) for i in range(rh)],
                  "rot": {"base": 200000.0, "dims": 128}}}}
    return {"architecture": "Vupolix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.25, "logit_scale": 0.25,
            "loop": {"start": 2, "stop": 4, "times": 2}, "layers": [time_mix, both] * 3, "max_positions": 16384, "eos_token_id": 2}


def vupolix_comparison(bw, torch, steps: int, dtype: str, only: str = "") -> int:
    """Prefill and decode of Vupolix at two layer sizes beside the Sepedra decoder (recurrent and attention layers over
    routed experts too) of equal width, depth and experts: one JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    for name, width, expert_ff in (("2048x(4x2048 of 32)", 2048, 2048), ("4096x(4x3584 of 32)", 4096, 3584)):
        for arch, cfg in (("Vupolix", vupolix_shape(width, expert_ff)), ("Sepedra", sepedra_shape(width, expert_ff, 2))):
            if only and only.lower() != arch.lower():
                continue
            model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            for tokens in (512, 2048):
                for exact in ((True, False) if arch == "Vupolix" else (True,)):
                    # (exact_cuts False: the matrix memories run a long portion in three passes over chunks)
                    m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens, exact_cuts=exact)
                    print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "prefill_tokens": tokens, "exact_cuts": exact,
                                      "ms": m["ms"], "tok_s": m["value"], "frac_of_matrix_peak": m["frac"]}), flush=True)
            for batch in (1, 8, 64):
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=2048)
                print(json.dumps({"shape": name, "model": arch, "dtype": dtype, "decode_batch": batch, "context": 2048,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
            del model
            torch.cuda.empty_cache()
    return 0


def sweep(bw, torch, steps: int, dtype: str) -> int:
    """Decode steps over batch and context, prefills over length: in bfloat16 at both shapes, in the 32-bit mode a
    coarser grid at the small one.  One JSON object a line."""
    from bitwise_amd.measure import PEAK_FLOPS, measure_decode, measure_prefill
    bf16 = dtype == "bfloat16"
    shapes = (("SmolLM2-1.7B", SMOLLM2_1_7B), ("Llama-3-8B", LLAMA3_8B)) if bf16 else (("SmolLM2-1.7B", SMOLLM2_1_7B),)
    for name, shape in shapes:
        cfg = dict(shape, max_position_embeddings=16384)
        model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
        for tokens in ((128, 256, 512, 1024, 2048) if bf16 else (128, 512, 2048)):
            m = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[dtype], tokens)
            print(json.dumps({"shape": name, "dtype": dtype, "prefill_tokens": tokens, "ms": m["ms"], "tok_s": m["value"],
                              "frac_of_matrix_peak": m["frac"]}), flush=True)
        for context in ((512, 2048, 8192) if bf16 else (512, 2048)):
            for batch in ((1, 2, 4, 8, 16, 32, 64, 128) if bf16 else (1, 8, 64)):
                if batch * context > 512 * 1024:          # (a pool of at most half a million tokens)
                    continue
                m = measure_decode(bw, torch, model, cfg, dtype, batch, steps, 4, context=context)
                print(json.dumps({"shape": name, "dtype": dtype, "decode_batch": batch, "context": context,
                                  "ms_per_step": m["ms_per_step"], "tok_s": m["tok_s"], "frac_of_8_TBs": m["roofline"]["frac"]}),
                      flush=True)
        del model
        torch.cuda.empty_cache()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has (named in config)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="the length of the headline prefill's prompt (for profiles of shorter prompts; up to 2048)")
    ap.add_argument("--shape", choices=["smollm2", "llama3_8b"], default="smollm2",
                    help="the layer sizes of the headline run (llama3_8b: for profiles of that shape; implies --no-points)")
    ap.add_argument("--trace-only", action="store_true",
                    help="run nothing but the 128-request shared-prefix trace at Llama-3-8B's sizes and print its figures (for profiles)")
    ap.add_argument("--decode-phases", action="store_true",
                    help="the headline decode with EngineConfig.decode_phases (its products as phases of a few launches; for profiles)")
    ap.add_argument("--portion-align", type=int, default=64,
                    help="EngineConfig.portion_align of the headline decode's engine (1: prompts cut exactly at the budget; for profiles)")
    ap.add_argument("--mixed", action="store_true",
                    help="only: an 8,192-token prompt beside 7 decoding requests, with portions cut at the budget and cut to whole blocks")
    ap.add_argument("--sweep", action="store_true",
                    help="print a table instead of the line: decode at batches 1 to 128 and contexts of 512 to 8,192 tokens, prefills "
                         "of 128 to 2,048 tokens, at both shapes (with --dtype fp32: a coarser grid at the small shape)")
    ap.add_argument("--sepedra", nargs="?", const="both", default="", choices=["both", "sepedra", "llama"],
                    help="print a table instead of the line: prefill and decode of the Sepedra design at two layer sizes beside "
                         "the Llama decoder of equal width and depth with a feed-forward as wide as a token's experts together")
    ap.add_argument("--vupolix", nargs="?", const="both", default="", choices=["both", "vupolix", "sepedra"],
                    help="print a table instead of the line: prefill and decode of the Vupolix design at two layer sizes beside "
                         "the Sepedra decoder of equal width, depth and experts (or one of the two)")
    ap.add_argument("--kikarax", nargs="?", const="both", default="", choices=["both", "kikarax", "llama"],
                    help="print a table instead of the line: prefill and decode of the Kikarax design at two layer sizes beside "
                         "the Llama decoder of equal width, depth and active feed-forward width (or one of the two only)")
    ap.add_argument("--kuponex", nargs="?", const="both", default="", choices=["both", "kuponex", "llama"],
                    help="print a table instead of the line: prefill and decode of the Kuponex design at two layer sizes beside "
                         "the Llama decoder of equal width, depth and feed-forward (or only one of the two)")
    ap.add_argument("--no-points", action="store_true",
                    help="only the headline: skip decode at batch 1 and 64, the 32-bit path and the Llama-3-8B sizes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported (use --gpus 1)")
        return 2

    import torch
    import bitwise_amd as bw
    from bitwise_amd.measure import (CONTEXT, PEAK_FLOPS, measure_chunked_prefill, measure_decode, measure_prefill, measure_serving,
                                     measure_trace)

    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    if args.sweep:
        return sweep(bw, torch, args.steps, dtype)
    if args.vupolix:
        return vupolix_comparison(bw, torch, min(args.steps, 32), dtype, "" if args.vupolix == "both" else args.vupolix)
    if args.kikarax:
        return kikarax_comparison(bw, torch, min(args.steps, 32), dtype, "" if args.kikarax == "both" else args.kikarax)
    if args.sepedra:
        return sepedra_comparison(bw, torch, min(args.steps, 32), dtype, "" if args.sepedra == "both" else args.sepedra)
    if args.kuponex:
        return kuponex_comparison(bw, torch, min(args.steps, 32), dtype, "" if args.kuponex == "both" else args.kuponex)
    if args.mixed:
        from bitwise_amd.measure import measure_prefill_beside_decodes, measure_qkv_row_orders
        cfg = dict(SMOLLM2_1_7B if args.shape == "smollm2" else LLAMA3_8B, max_position_embeddings=16384)
        model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
        print(json.dumps({"shape": args.shape, "dtype": args.dtype,
                          "prompt_beside_decodes": [measure_prefill_beside_decodes(bw, torch, model, cfg, dtype, portion_align=a)
                                                    for a in (1, 64, 1, 64)],
                          "qkv_us_by_row_order": measure_qkv_row_orders(torch, cfg) if args.dtype == "bf16" else {}}))
        return 0
    if args.trace_only:
        big = dict(LLAMA3_8B, max_position_embeddings=16384)
        model8 = bw.Model.random(big, seed=1, dtype=dtype, sigma=0.02, on_device=True)
        print(json.dumps({"llama3_8b.trace8k": measure_trace(bw, torch, model8, big, dtype, check=8), "dtype": args.dtype}))
        return 0
    cfg = dict(SMOLLM2_1_7B if args.shape == "smollm2" else LLAMA3_8B)
    shape_name = "SmolLM2-1.7B" if args.shape == "smollm2" else "Llama-3-8B"
    if args.shape != "smollm2":
        args.no_points = True
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    t_start = time.perf_counter()
    model = bw.Model.random(cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
    vocab = cfg["vocab_size"]
    side_steps = max(16, args.steps // 2)

    if not 1 <= args.prefill_tokens <= PREFILL_TOKENS:
        print(f"bench.py: --prefill-tokens {args.prefill_tokens} is outside 1..{PREFILL_TOKENS}")
        return 2
    prefill = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[args.dtype], args.prefill_tokens)
    head = measure_decode(bw, torch, model, cfg, dtype, args.batch, args.steps, args.warmup, decode_phases=args.decode_phases,
                         portion_align=args.portion_align)
    points, point_rooflines = {}, {}
    extra = {}
    if not args.no_points:
        for b in (1, 64):
            m = measure_decode(bw, torch, model, cfg, dtype, b, side_steps, 4)
            points[f"decode_b{b}"] = m["tok_s"]
            point_rooflines[f"decode_b{b}"] = m["roofline"]
        for t in (128, 512):                          # shorter prompts, one step each: tokens a second
            points[f"prefill_t{t}"] = measure_prefill(bw, torch, model, cfg, dtype, PEAK_FLOPS[args.dtype], t)["value"]
        if args.dtype == "bf16":
            # the same layers with 8,192-token contexts (position tables of 16,384; batch 8)
            del model
            torch.cuda.empty_cache()
            long_cfg = dict(cfg, max_position_embeddings=16384)
            model_long = bw.Model.random(long_cfg, seed=0, dtype=dtype, sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model_long, long_cfg, dtype, 8, side_steps, 4, context=8192)
            points["decode_b8_ctx8192"] = m["tok_s"]
            point_rooflines["decode_b8_ctx8192"] = m["roofline"]
            del model_long
            model = None
            torch.cuda.empty_cache()
            # the true 32-bit path of the same model (the same bfloat16 weights, widened exactly; 32-bit caches)
            model32 = bw.Model.random(cfg, seed=0, dtype="float32", sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model32, cfg, "float32", args.batch, side_steps, 4)
            extra["fp32"] = {"decode_tok_s": m["tok_s"], "batch": args.batch, "ms_per_step": m["ms_per_step"],
                             "roofline": m["roofline"], "weights_stored_as": "bfloat16, widened exactly where they are used",
                             "prefill": measure_prefill(bw, torch, model32, cfg, "float32", PEAK_FLOPS["fp32"])}
            del model32
            torch.cuda.empty_cache()
            # Llama-3-8B's sizes, all 32 layers, bfloat16 (position tables of 16,384 for the 8,192-token contexts): decode at
            # batch 8, 1 and 64 with 2,048-token contexts and at batch 8 with 8,192-token contexts, a prefill of 2,048 tokens
            # in one step and one of 8,192 in portions of 2,048
            big = dict(LLAMA3_8B, max_position_embeddings=16384)
            model8 = bw.Model.random(big, seed=1, dtype="bfloat16", sigma=0.02, on_device=True)
            m = measure_decode(bw, torch, model8, big, "bfloat16", 8, side_steps, 4)
            points8, rooflines8 = {}, {}
            for name, b, ctx in (("decode_b1", 1, CONTEXT), ("decode_b64", 64, CONTEXT), ("decode_b8_ctx8192", 8, 8192)):
                mp = measure_decode(bw, torch, model8, big, "bfloat16", b, side_steps, 4, context=ctx)
                points8[name] = mp["tok_s"]
                rooflines8[name] = mp["roofline"]["frac"]
            extra["llama3_8b"] = {"layers": big["num_hidden_layers"], "hidden": big["hidden_size"], "heads": 32, "kv_heads": 8,
                                  "head_dim": 128, "ffn": big["intermediate_size"], "vocab": big["vocab_size"],
                                  "decode_tok_s": m["tok_s"], "batch": 8, "ms_per_step": m["ms_per_step"],
                                  "roofline": m["roofline"], "points": points8, "point_roofline_fracs": rooflines8,
                                  "prefill": measure_prefill(bw, torch, model8, big, "bfloat16", PEAK_FLOPS["bf16"]),
                                  "prefill_8192_in_portions": measure_chunked_prefill(bw, torch, model8, big, "bfloat16",
                                                                                      PEAK_FLOPS["bf16"]),
                                  "serving": measure_serving(bw, torch, model8, big, "bfloat16"),
                                  # 128 requests, four shared 1,024-token starts, contexts up to 6,144, a tenth cancelled, a pool
                                  # that forces preemption; 8 of them checked against solo runs
                                  "trace8k": measure_trace(bw, torch, model8, big, "bfloat16", check=8)}
            del model8
            model = None

    value = head["tok_s"]
    # The reference's figure is one stream on a CPU: like for like is this engine's rate at batch 1, where it is measured.
    one_stream = points.get("decode_b1", value if args.batch == 1 else None)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {shape_name} shape, 2048-token contexts",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / BASELINE_TOK_S, 1) if args.shape == "smollm2" else None,
        "vs_baseline_one_stream": round(one_stream / BASELINE_TOK_S, 1) if args.shape == "smollm2" and one_stream else None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {
            "model": f"{shape_name} shape, random weights", "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"], "ffn": cfg["intermediate_size"],
            "vocab": vocab, "tied": bool(cfg["tie_word_embeddings"]), "global_batch": args.batch, "seq_len": CONTEXT, "max_context": 4096,
            "page_size": 16, "parallelism": "single GPU", "weights": "bf16" if args.dtype == "bf16" else "bf16 widened",
            "baseline": f"reference CPU decode, one stream, 7.26 tok/s (vs_baseline: batch {args.batch} over it)",
        },
        "prefill": prefill,
        "roofline": head["roofline"],
        "points": points,
        "point_rooflines": point_rooflines,
    }
    line.update(extra)
    line["wall_s"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
