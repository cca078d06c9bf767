#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

Default: the LLaMA-2-7B layer sizes (32 layers, hidden 4096, 32/32 heads of 128,
feed-forward 11008, vocabulary 32000) with seeded random bfloat16 weights, a batch
of 8 sequences with 512-token prompts that decode 256 tokens (8 more to warm up),
cache context 4096.  A step is one decode step of the whole batch: step function, greedy choice on the device, the tokens
back on the host.  One JSON line is printed: decoded tokens per second, the
prefill of 2,048 tokens, the decode step against the HBM roofline, and decoding
at batch 1 and 64.  Peaks are the published ones of MI355X (HBM 8 TB/s, dense
bf16 MFMA 2.5 PFLOP/s, float32 157.3 TFLOP/s).
"""
import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA2_7B = {"architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": 11008,
             "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 32,
             "vocab_size": 32000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
             "max_position_embeddings": 4096, "tie_word_embeddings": False,
             "bos_token_id": 1, "eos_token_id": 2}


LLAMA3_8B = dict(LLAMA2_7B, intermediate_size=14336, num_key_value_heads=8, vocab_size=128256,
                 rope_theta=500000.0, max_position_embeddings=8192)
LLAMA2_70B = dict(LLAMA2_7B, hidden_size=8192, intermediate_size=28672, num_hidden_layers=80,
                  num_attention_heads=64, num_key_value_heads=8)
SHAPES = {"llama2-7b": ("LLaMA-2-7B shape", LLAMA2_7B), "llama3-8b": ("LLaMA-3-8B shape", LLAMA3_8B),
          "llama2-70b": ("LLaMA-2-70B shape", LLAMA2_70B)}


def weight_bytes_per_step(cfg, layers, esz):
    E, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", E // nh)
    per_layer = ((nh + 2 * nkv) * hd * E + E * nh * hd + 3 * E * F + 2 * E) * esz
    return layers * per_layer + (V * E + E) * esz


def kv_bytes_per_token(cfg, layers, esz):
    nkv = cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    return layers * 2 * nkv * hd * esz


def prefill_flops(cfg, layers, T, out_rows=1):
    E, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", E // nh)
    linear = 2.0 * T * ((nh + 2 * nkv) * hd * E + E * nh * hd + 3 * E * F)
    attn = 2.0 * 2.0 * nh * hd * (T * (T + 1) / 2)
    return layers * (linear + attn) + 2.0 * out_rows * V * E


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--shape", default="llama2-7b", choices=sorted(SHAPES),
                    help="layer sizes (default: the headline configuration)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiles); prints its own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only (this library has no multi-GPU path); --gpus must be 1")
        return 2

    import torch
    from inferllm_amd import Engine, StepEntry
    from inferllm_amd.kernels import ops
    from inferllm_amd.sampling import Sampler, SamplingParams

    shape_name, shape_cfg = SHAPES[args.shape]
    cfg = dict(shape_cfg)
    full_layers = cfg["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg["num_hidden_layers"] = layers
    ctx_len = cfg["max_position_embeddings"]
    esz = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    dev = "cuda:0"
    max_b = max(args.batch, 1 if args.no_points else 64)
    per_seq = -(-(args.prompt + args.steps + args.warmup + 2) // 64) * 64     # whole cache pages
    room = max(max_b * max(per_seq, 1024), 4096)
    t0 = time.time()
    eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, device=dev, max_batch=max_b,
                             max_seq_len=ctx_len, max_tokens=room)
    torch.cuda.synchronize()
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    g = torch.Generator().manual_seed(1234)

    def decode_run(batch, steps, warmup):
        """tokens/s, ms/step, mean context of `steps` timed decode steps of `batch` sequences."""
        prompts = [torch.randint(0, cfg["vocab_size"], (args.prompt,), generator=g).tolist()
                   for _ in range(batch)]
        slots = [eng.alloc_slot() for _ in range(batch)]
        # prompts go in pieces of at most 8 sequences to bound the prefill's activations
        toks = [0] * batch
        for i in range(0, batch, 8):
            part = list(range(i, min(batch, i + 8)))
            logits = eng.step([StepEntry(slots[j], prompts[j], [args.prompt - 1]) for j in part])
            for j, t in zip(part, ops.argmax(logits.contiguous()).tolist()):
                toks[j] = t

        # as the generation loop runs greedy requests: a step starts from the tokens the last
        # one chose on the device, and the host reads every step's tokens while the next runs
        sampler = Sampler(SamplingParams(), eng.device)             # greedy
        draw = sampler.draw(eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)]),
                            [0] * batch, [0] * batch)

        seen = []

        def one():
            nonlocal draw
            logits = eng.step([StepEntry(s, [0], [0]) for s in slots], device_tokens=draw.device)
            following = sampler.draw(logits, [0] * batch, [0] * batch)
            seen.append(draw.tokens())
            draw = following
            return logits

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            logits = one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        # what was timed must have computed something: finite logits, and greedy tokens that
        # change from step to step (a run on NaN or constant logits would be as fast)
        if not bool(torch.isfinite(logits).all()):
            raise SystemExit(f"bench: non-finite logits in the decode run at batch {batch}")
        distinct = {int(t) for row in seen for t in row}
        print(f"[bench] batch {batch}: {len(distinct)} distinct greedy tokens in {len(seen)} steps",
              file=sys.stderr, flush=True)
        if len(seen) >= 16 and len(distinct) < 2:
            raise SystemExit(f"bench: the greedy token is {sorted(distinct)} in every step of every "
                             f"sequence at batch {batch}: the logits are degenerate")
        mean_ctx = args.prompt + 1 + warmup + (steps + 1) / 2.0
        for s in slots:
            eng.free_slot(s)
        return batch * steps / dt, dt / steps * 1e3, mean_ctx

    def prefill_run(T=2048, reps=3):
        ids = torch.randint(0, cfg["vocab_size"], (T,), generator=g).tolist()
        times = []
        for i in range(reps):
            s = eng.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = eng.step([StepEntry(s, ids, [T - 1])])
            ops.argmax(logits).tolist()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            if not bool(torch.isfinite(logits).all()):
                raise SystemExit("bench: non-finite logits in the prefill")
            eng.free_slot(s)
        pt = min(times[1:])
        fl = prefill_flops(cfg, layers, T)
        return {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                "frac": round(fl / pt / (PEAK_TFLOPS[dkey] * 1e12), 4)}

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_run(reps=max(3, args.steps))}), flush=True)
        return 0

    tps, ms, mean_ctx = decode_run(args.batch, args.steps, args.warmup)
    step_bytes = weight_bytes_per_step(cfg, layers, esz) + args.batch * mean_ctx * kv_bytes_per_token(cfg, layers, esz)
    achieved = step_bytes / (ms * 1e-3) / 1e9
    out = {
        "metric": "decode tok/s at batch 1/8/64 + prefill tok/s at 2,048 tokens (LLaMA-2-7B)",
        "value_is": f"decode tokens/s at batch {args.batch}", "value": round(tps, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic: seeded random weights N(0, 0.02), uniform random token ids",
        "config": {"model": shape_name, "layers": layers, "layers_full": full_layers,
                   "hidden_size": cfg["hidden_size"], "intermediate_size": cfg["intermediate_size"],
                   "num_attention_heads": cfg["num_attention_heads"],
                   "num_key_value_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]),
                   "vocab_size": cfg["vocab_size"], "global_batch": args.batch,
                   "seq_len": ctx_len, "prompt_len": args.prompt, "rope_theta": cfg["rope_theta"],
                   "rms_norm_eps": cfg["rms_norm_eps"], "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        out["prefill"] = prefill_run()
        b1, _, _ = decode_run(1, min(args.steps, 256), 4)
        b64, _, _ = decode_run(64, min(args.steps, 256), 4)
        out["points"] = {"decode_b1": round(b1, 2), "decode_b64": round(b64, 2)}
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
