#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

Default: the LLaMA-2-7B layer sizes (32 layers, hidden 4096, 32/32 heads of 128,
feed-forward 11008, vocabulary 32000) with seeded random bfloat16 weights, a batch
of 8 sequences with 512-token prompts that decode 256 tokens (8 more to warm up),
cache context 4096.  A step is one decode step of the whole batch: step function, greedy choice on the device, the tokens
back on the host, as `Engine.generate` runs it.  One JSON line is printed: decoded tokens per second, the
prefill of 2,048 tokens, the decode step against the HBM roofline, and under
`points` decoding at batch 1 and 64, decoding from 3,800-token contexts at batch
8 and 64, milliseconds to the first token of prompts of 16, 64 and 160 tokens, prefills of
64 x 128, 8,192 and 16,384 tokens (and of 16,384 in steps of 2,048 that go on from the paged
cache), the LLaMA-3-8B shape with 16 prompts of 64 to 4,096 tokens and with 8 sequences at
8,000-token contexts, and the LLaMA-2-70B shape (prefill of 2,048 tokens, decode at batch 1 and
32 from 1,024-token prompts; `--no-70b` leaves it out).  Every decode run goes through the
engine's generation loop, whose stopwatch starts after the warm-up steps.  Every decode point has a
`..._hbm_frac` beside it: the bytes its step has to read (every weight once, the
cache of its live sequences) / its time / the HBM peak.  Peaks are the published ones
of MI355X (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, float32 157.3 TFLOP/s).
The run fails (non-zero) if any timed run produced a non-finite logit or the same
greedy token everywhere.
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


def prefill_flops(cfg, layers, T, out_rows=1, lens=None):
    """Flops of a prefill of T tokens (`lens`: the prompts' lengths if more than one)."""
    E, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim", E // nh)
    linear = 2.0 * T * ((nh + 2 * nkv) * hd * E + E * nh * hd + 3 * E * F)
    attn = sum(2.0 * 2.0 * nh * hd * (n * (n + 1) / 2) for n in (lens or [T]))
    return layers * (linear + attn) + 2.0 * out_rows * V * E


class Bench:
    """One engine of one shape and the runs on it."""

    def __init__(self, cfg, layers, dtype, max_batch, max_tokens, seed=1234):
        import torch
        from inferllm_amd import Engine
        self.torch = torch
        self.cfg = dict(cfg)
        self.full_layers = cfg["num_hidden_layers"]
        self.layers = layers or self.full_layers
        self.cfg["num_hidden_layers"] = self.layers
        self.esz = 2 if dtype == "bfloat16" else 4
        self.dkey = "bf16" if dtype == "bfloat16" else "fp32"
        t0 = time.time()
        self.eng = Engine.from_random(self.cfg, seed=0, dtype=dtype, device="cuda:0",
                                      max_batch=max_batch, max_seq_len=cfg["max_position_embeddings"],
                                      max_tokens=max_tokens)
        torch.cuda.synchronize()
        print(f"[bench] engine ready in {time.time() - t0:.1f} s "
              f"({self.layers} layers, room for {max_tokens} tokens)", file=sys.stderr, flush=True)
        self.g = torch.Generator().manual_seed(seed)

    def close(self):
        self.eng = None
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    def ids(self, n):
        return self.torch.randint(0, self.cfg["vocab_size"], (n,), generator=self.g).tolist()

    def step_bytes(self, batch, mean_ctx):
        return (weight_bytes_per_step(self.cfg, self.layers, self.esz)
                + batch * mean_ctx * kv_bytes_per_token(self.cfg, self.layers, self.esz))

    def decode_run(self, batch, steps, warmup, prompt):
        """(tokens/s, ms/step, fraction of the HBM peak) of `steps` timed decode steps of `batch`
        sequences that start from prompts of `prompt` tokens, through the engine's generation
        loop (greedy, no stop token): the loop runs `warmup` decode steps, waits for the device,
        and its stopwatch runs from there to the end of the batch."""
        from inferllm_amd.sampling import Sampler, SamplingParams
        torch, eng = self.torch, self.eng
        prompts = [self.ids(prompt) for _ in range(batch)]
        params = SamplingParams()                                   # greedy
        # (prompts go in steps of at most 16,384 tokens to bound the prefill's activations)
        loop = eng.generation_loop(Sampler(params, eng.device), max_step_tokens=16384)
        loop.time_after = warmup
        out = loop.run(prompts, params, warmup + steps + 1, [])
        st = loop.stats
        if st.timed_steps != steps or st.batches != 1 or any(len(o) != warmup + steps + 1 for o in out):
            raise SystemExit(f"bench: the loop timed {st.timed_steps} steps of {st.batches} batches at "
                             f"batch {batch}, not {steps} of one")
        dt = st.timed_seconds
        # what was timed must have computed something: greedy tokens that are not one and the same
        # everywhere (a run on NaN or constant logits would be as fast)
        distinct = {int(t) for o in out for t in o}
        print(f"[bench] batch {batch}, prompts of {prompt}: {dt / steps * 1e3:.3f} ms a step, "
              f"{len(distinct)} distinct greedy tokens in {steps + warmup} steps", file=sys.stderr, flush=True)
        if steps + warmup >= 16 and len(distinct) < 2:
            raise SystemExit(f"bench: the greedy token is {sorted(distinct)} in every step of every "
                             f"sequence at batch {batch}: the logits are degenerate")
        mean_ctx = prompt + 1 + warmup + (steps + 1) / 2.0
        ms = dt / steps * 1e3
        frac = self.step_bytes(batch, mean_ctx) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        return batch * steps / dt, ms, frac

    def prefill_run(self, T=2048, reps=6, prompts=1, max_step_tokens=None, skip=1):
        """`prompts` prompts of T tokens each in one step (or, with `max_step_tokens`, one prompt in
        steps of that many tokens that go on from the cache): tokens/s of the fastest of `reps` runs
        after the first `skip`, the time to the first token in ms, and the fraction of the matrix peak."""
        from inferllm_amd import StepEntry
        from inferllm_amd.kernels import ops
        torch, eng = self.torch, self.eng
        ids = [self.ids(T) for _ in range(prompts)]
        times = []
        for i in range(reps):
            slots = [eng.alloc_slot() for _ in ids]
            torch.cuda.synchronize()
            t = time.perf_counter()
            if max_step_tokens is None:
                logits = eng.step([StepEntry(s, p, [T - 1]) for s, p in zip(slots, ids)])
            else:
                for a in range(0, T, max_step_tokens):
                    piece = ids[0][a:a + max_step_tokens]
                    logits = eng.step([StepEntry(slots[0], piece, [len(piece) - 1] if a + len(piece) == T else [])])
            ops.argmax(logits).tolist()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            if not bool(torch.isfinite(logits).all()):
                raise SystemExit("bench: non-finite logits in the prefill")
            for s in slots:
                eng.free_slot(s)
        pt = min(times[skip:])
        fl = prefill_flops(self.cfg, self.layers, T * prompts, prompts, [T] * prompts)
        return {"value": round(T * prompts / pt, 1), "tokens": T * prompts, "ms": round(pt * 1e3, 3),
                "frac": round(fl / pt / (PEAK_TFLOPS[self.dkey] * 1e12), 4)}

    def generate_run(self, lens, new_tokens):
        """Prompts of the given lengths through `Engine.generate` (all in one batch), three times
        (the first sets libraries and graphs up, the second may still take fresh memory from the
        driver for what the graphs' pools cannot lend it); the third run's figures: (prefill
        tokens/s, its fraction of the matrix peak, decode tokens/s, its fraction of the HBM peak)."""
        prompts = [self.ids(n) for n in lens]
        for _ in range(3):
            out = self.eng.generate(prompts, max_new_tokens=new_tokens, stop_token_ids=[])
            st = self.eng.last_stats
        assert all(len(o) == new_tokens for o in out)
        if len({t for o in out for t in o}) < 2:
            raise SystemExit("bench: the generation loop produced one and the same token everywhere")
        B, T = len(lens), sum(lens)
        pf = T / st.prefill_seconds
        pf_frac = (prefill_flops(self.cfg, self.layers, T, B, lens) / st.prefill_seconds
                   / (PEAK_TFLOPS[self.dkey] * 1e12))
        steps = st.decode_steps
        ms = st.decode_seconds / steps * 1e3
        mean_ctx = T / B + 1 + (steps + 1) / 2.0
        frac = self.step_bytes(B, mean_ctx) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        return pf, pf_frac, B * steps / st.decode_seconds, frac


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
    ap.add_argument("--no-points", action="store_true", help="skip everything under `points` and the prefill")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiles); prints its own line")
    ap.add_argument("--no-70b", action="store_true",
                    help="leave the LLaMA-2-70B shape out of `points` (138 GB of weights: half a minute)")
    ap.add_argument("--with-70b", action="store_true", help="(the default now; kept for old command lines)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only (this library has no multi-GPU path); --gpus must be 1")
        return 2

    shape_name, shape_cfg = SHAPES[args.shape]
    ctx_len = shape_cfg["max_position_embeddings"]
    headline = args.shape == "llama2-7b" and args.dtype == "bfloat16" and not args.no_points
    long_ctx = 3800
    max_b = max(args.batch, 1 if args.no_points else (128 if headline else 64))
    per_seq = -(-(args.prompt + args.steps + args.warmup + 2) // 64) * 64     # whole cache pages
    room = max(max_b * max(per_seq, 1024), 4096)
    if headline:
        room = max(room, 64 * (-(-(long_ctx + 64 + 8) // 64) * 64))
    b = Bench(shape_cfg, args.layers, args.dtype, max_b, room)
    cfg, layers = b.cfg, b.layers

    if args.prefill_only:
        print(json.dumps({"prefill": b.prefill_run(reps=max(3, args.steps))}), flush=True)
        return 0

    tps, ms, frac = b.decode_run(args.batch, args.steps, args.warmup, args.prompt)
    out = {
        "metric": "decode tok/s at batch 1/8/64 + prefill tok/s at 2,048 tokens (LLaMA-2-7B)",
        "value_is": f"decode tokens/s at batch {args.batch}", "value": round(tps, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": b.dkey, "data": "synthetic: seeded random weights N(0, 0.02), uniform random token ids",
        "config": {"model": shape_name, "layers": layers, "layers_full": b.full_layers,
                   "hidden_size": cfg["hidden_size"], "intermediate_size": cfg["intermediate_size"],
                   "num_attention_heads": cfg["num_attention_heads"],
                   "num_key_value_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]),
                   "vocab_size": cfg["vocab_size"], "global_batch": args.batch,
                   "seq_len": ctx_len, "prompt_len": args.prompt, "rope_theta": cfg["rope_theta"],
                   "rms_norm_eps": cfg["rms_norm_eps"], "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(frac * HBM_PEAK_GBS, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(frac, 4)},
    }
    if not args.no_points:
        out["prefill"] = b.prefill_run()
        points = {}
        few = min(args.steps, 256)
        for name, batch in (("decode_b1", 1), ("decode_b64", 64)):
            v, _, f = b.decode_run(batch, few, 4, args.prompt)
            points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
        if headline:
            v, _, f = b.decode_run(128, 64, 4, args.prompt)
            points["decode_b128"], points["decode_b128_hbm_frac"] = round(v, 2), round(f, 4)
            # long contexts: the cache's share of a step's bytes grows from a seventh to nine tenths
            for name, batch in (("decode_b8_ctx3800", 8), ("decode_b64_ctx3800", 64)):
                v, _, f = b.decode_run(batch, 64, 4, long_ctx)
                points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
            # short prompts: milliseconds to the first token (their steps are replayed from graphs
            # from the second of a shape on), and 64 prompts of 128 tokens in one step
            for n in (16, 64, 160):
                points[f"first_token_ms_prompt{n}"] = b.prefill_run(n, reps=8, skip=3)["ms"]
            p = b.prefill_run(128, prompts=64)
            points["prefill_64x128"], points["prefill_64x128_frac"] = p["value"], p["frac"]
            b.close()
            # the same layer sizes with room for 16,384 positions: one long prompt whole, and in
            # steps of 2,048 tokens that go on from the paged cache
            long = Bench(dict(LLAMA2_7B, max_position_embeddings=16384), args.layers, args.dtype, 1, 16384 + 64)
            for T in (8192, 16384):
                p = long.prefill_run(T, reps=3)
                points[f"prefill_{T}"], points[f"prefill_{T}_frac"] = p["value"], p["frac"]
            p = long.prefill_run(16384, reps=3, max_step_tokens=2048)
            points["prefill_16384_in_steps_of_2048"], points["prefill_16384_in_steps_of_2048_frac"] = p["value"], p["frac"]
            long.close()
            # LLaMA-3-8B shape (grouped heads, vocabulary 128,256): 16 prompts of 64 to 4,096
            # tokens, lengths seeded, one batch through the generation loop, 128 new tokens each;
            # and 8 sequences decoding from 8,000-token contexts (its context is 8,192)
            import torch
            lens = torch.randint(64, 4097, (16,), generator=torch.Generator().manual_seed(16)).tolist()
            total = max(sum(-(-(n + 130) // 64) * 64 for n in lens), 8 * 8192)
            b8 = Bench(LLAMA3_8B, 0, args.dtype, 16, total)
            pf, pf_frac, dc, dc_frac = b8.generate_run(lens, 128)
            points.update({"llama3_8b_ragged16_prompt_tokens": sum(lens),
                           "llama3_8b_ragged16_prefill": round(pf, 1),
                           "llama3_8b_ragged16_prefill_frac": round(pf_frac, 4),
                           "llama3_8b_ragged16_decode": round(dc, 2),
                           "llama3_8b_ragged16_decode_hbm_frac": round(dc_frac, 4)})
            v, _, f = b8.decode_run(8, 64, 4, 8000)
            points["llama3_8b_decode_b8_ctx8000"], points["llama3_8b_decode_b8_ctx8000_hbm_frac"] = round(v, 2), round(f, 4)
            b8.close()
            if not args.no_70b:
                b70 = Bench(LLAMA2_70B, 0, args.dtype, 32, 32 * 1280)
                p70 = b70.prefill_run()
                points.update({"llama2_70b_prefill": p70["value"], "llama2_70b_prefill_frac": p70["frac"]})
                for name, batch in (("llama2_70b_decode_b1", 1), ("llama2_70b_decode_b32", 32)):
                    v, _, f = b70.decode_run(batch, 128, 4, 1024)
                    points[name], points[name + "_hbm_frac"] = round(v, 2), round(f, 4)
                b70.close()
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
