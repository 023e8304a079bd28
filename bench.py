#!/usr/bin/env python3
"""Benchmark of the CASTLE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-decode] [--no-lm] [--no-cpu]

Workload (benchmark configuration 2): one Castle layer (dim 512, 8 heads, dim_head 64), bf16,
x and the upstream gradient ~ N(0,1) of shape (4, 4096, 512), seeded random-init weights;
one step = forward + backward of the layer (projection GEMMs included), inputs resident in
HBM.  Prints ONE JSON line:
  value        layer TFLOP/s = (19*B*H*L^2*d core flop + projection GEMM flop) / step time
  core         the same for the attention core alone, from per-kernel HIP-event times
  roofline     the longest-running kernel against the bf16 MFMA peak (2.5 PFLOP/s)
  decode       benchmark configuration 4 (B32, prefill 2048, 512 cached steps): tokens/s and the decode
               stream kernel against the HBM peak (8 TB/s)
  lm           benchmark configuration 5 (12 x [Castle + MLP], tied embedding, (16, 1024) tokens, bf16): one
               forward + loss + backward, and greedy generation through prefill + cached decode
  cpu_baseline the CPU oracle (dense PyTorch restatement of the reference's non-Triton path)
               on a bounded sample of the same workload, host cores stated
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16/fp16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "castle_cfg2_cfg4_pmc_hbm_traffic.txt")


def recorded_traffic():
    """HBM bytes per launch of the config 2 / config 4 kernels as recorded in the rocprofv3 summary
    under profiles/ (FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy; its last line is a JSON object
    written with the table).  These are recorded counters, not something this script measures: the
    line names the file and the commit the counters were collected at.  {} when the file is absent."""
    try:
        with open(TRAFFIC_PROFILE) as fh:
            tail = [l for l in fh if l.startswith("# json: ")]
        return json.loads(tail[-1][len("# json: "):]) if tail else {}
    except (OSError, ValueError):
        return {}


# algorithmic contractions (unit: B*H*L^2*d flop = 2*d flop per causal pair) attributed to each kernel.
# They sum to 18: the 19th contraction of the algorithmic count (the forward state update, which a
# backward pass that keeps nothing would repeat) is not executed because the snapshots are kept.
KERNEL_UNITS = {"prep": 0.0, "scan": 2.0, "attn": 3.0, "delta": 0.0, "bwd_key": 9.0, "bwd_query": 4.0}


def cfg2_flops(B, H, L, d, dim):
    unit = float(B) * H * L * L * d
    core = 19.0 * unit
    gemm = 3.0 * (2.0 * B * L * dim * 6 * H * d + 2.0 * B * L * H * d * dim)
    return unit, core, gemm


def bench_layer(steps, warmup):
    import torch

    from lookahead_keys_attention_amd import Castle, _native

    dev = torch.device("cuda:0")
    B, L, dim, H, d = 4, 4096, 512, 8, 64
    torch.manual_seed(0)
    model = Castle(dim, heads=H, dim_head=d, use_triton=True).to(dev).bfloat16()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, L, dim, generator=g).bfloat16().to(dev).requires_grad_()
    gy = torch.randn(B, L, dim, generator=g).bfloat16().to(dev)

    def step():
        model.zero_grad(set_to_none=True)
        x.grad = None
        y = model(x)
        y.backward(gy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    # per-kernel durations: HIP events recorded by the library on the launch stream
    _native.profile_enable(True)
    for _ in range(steps):
        step()
    records = _native.profile_read()
    _native.profile_enable(False)
    per = {}
    for name, ms in records:
        per.setdefault(name, []).append(ms)
    kernels = {k: sum(v) / len(v) for k, v in per.items()}
    unit, core, gemm = cfg2_flops(B, H, L, d, dim)
    core_ms = sum(kernels.values())
    table = {k: {"ms": round(v, 4), "tflops": round(KERNEL_UNITS[k] * unit / (v * 1e-3) / 1e12, 2)} for k, v in kernels.items()}
    dom = max(kernels, key=kernels.get)
    achieved = KERNEL_UNITS[dom] * unit / (kernels[dom] * 1e-3) / 1e12
    rec = recorded_traffic()
    traffic = rec.get("bytes", {})
    code = N_lib_code_ints(B, H, L, d)
    executed = sum(KERNEL_UNITS.values()) * unit
    return {
        "ms_per_step": ms_per_step,
        "value": (core + gemm) / (ms_per_step * 1e-3) / 1e12,
        # flop: the algorithmic count 19*B*H*L^2*d of the metric; the kernels are charged 18 of those units
        "core": {"flop": core, "ms": round(core_ms, 4), "tflops": round(core / (core_ms * 1e-3) / 1e12, 2),
                 "frac_of_peak": round(core / (core_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                 "tflops_18_units": round(executed / (core_ms * 1e-3) / 1e12, 2),
                 "frac_of_peak_18_units": round(executed / (core_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                 "kernels": table, "workspace_bytes": code},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": traffic.get(dom),
                     "traffic_source": rec.get("source"),
                     # the same launch seen from the memory side: recorded HBM bytes / live duration
                     "hbm_GBps": round(traffic[dom] / (table[dom]["ms"] * 1e-3) / 1e9, 1) if dom in traffic else None,
                     "hbm_frac": round(traffic[dom] / (table[dom]["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4) if dom in traffic else None},
        "global_batch": B, "seq_len": L,
    }


def N_lib_code_ints(B, H, L, d, dtype_code=1):
    """Device bytes one forward + backward call holds: kept for backward, forward state, backward transient."""
    from lookahead_keys_attention_amd import _native

    lib = _native.lib()
    return {"kept_for_backward": int(lib.castle_fwd_workspace_bytes(B, H, L, d, dtype_code)),
            "forward_state": int(lib.castle_fwd_state_bytes(B, H, L, d, dtype_code)),
            "backward_transient": int(lib.castle_bwd_workspace_bytes(B, H, L, d, dtype_code, 0))}


def bench_long_context(steps=3, warmup=2):
    """Benchmark configuration 3: one Castle layer forward+backward, dim 2048, 16 heads, dim_head 128,
    batch 1, seq 16384, bf16.  About 27 GB of workspace (see workspace_bytes); --no-long-context skips it."""
    import torch

    from lookahead_keys_attention_amd import Castle, _native

    dev = torch.device("cuda:0")
    B, L, dim, H, d = 1, 16384, 2048, 16, 128
    torch.manual_seed(0)
    model = Castle(dim, heads=H, dim_head=d, use_triton=True).to(dev).bfloat16()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, L, dim, generator=g).bfloat16().to(dev).requires_grad_()
    gy = torch.randn(B, L, dim, generator=g).bfloat16().to(dev)

    def step():
        model.zero_grad(set_to_none=True)
        x.grad = None
        model(x).backward(gy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    _native.profile_enable(True)
    step()
    records = _native.profile_read()
    _native.profile_enable(False)
    per = {}
    for name, t in records:   # the d = 128 backward launches each kernel twice: summed per slot
        per[name] = per.get(name, 0.0) + t
    _, core, _ = cfg2_flops(B, H, L, d, dim)
    core_ms = sum(per.values())
    return {"workload": "config 3: one Castle layer forward+backward, dim 2048, 16 heads, dim_head 128, batch 1, "
                        "seq 16384, bf16 tensors",
            "ms_per_step": round(ms, 3), "core_ms": round(core_ms, 3),
            "core_tflops": round(core / (core_ms * 1e-3) / 1e12, 2),
            "frac_of_peak": round(core / (core_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
            "kernels_ms": {k: round(v, 3) for k, v in per.items()},
            "workspace_bytes": N_lib_code_ints(B, H, L, d)}


def decode_step_bytes(B, H, t, d, es, base, defer=4):
    """HBM bytes one cached step moves at row count t with the deferred write-back: the four cached
    rows read, the cached gates (16 bytes per row) read while tokens are pending, the lookahead keys
    written on every `defer`-th step and one gate (4 bytes) per row on the others, the new rows."""
    pending = t - max(base, t - t % defer)
    per_row = 4 * d * es + (4 * defer if pending > 0 else 0) + (d * es if (t + 1) % defer == 0 else 4)
    return B * H * (t * per_row + 8 * d * es)


def bench_decode(n_steps=512, prefill=2048):
    import torch

    from lookahead_keys_attention_amd import Castle, _native

    dev = torch.device("cuda:0")
    B, dim, H, d = 32, 512, 8, 64
    torch.manual_seed(0)
    model = Castle(dim, heads=H, dim_head=d, use_triton=True).to(dev).bfloat16().eval()
    g = torch.Generator().manual_seed(1)
    x0 = torch.randn(B, prefill, dim, generator=g).bfloat16().to(dev)
    xs = torch.randn(B, n_steps, dim, generator=g).bfloat16().to(dev)
    out = {}
    with torch.no_grad():
        for timed in (False, True):            # first round warms up, second is timed
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            _, cache = model(x0, return_next_cache=True)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for t in range(n_steps):
                _, cache = model(xs[:, t:t + 1], cache=cache)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
        out["prefill_tokens_per_s"] = B * prefill / (t1 - t0)
        out["tokens_per_s"] = B * n_steps / (t2 - t1)
        out["ms_per_decode_step"] = (t2 - t1) * 1e3 / n_steps
        # kernel-level: bytes the stream kernel must move per step, B*H*(5*t*d + 8*d)*2, against its duration
        _, cache = model(x0, return_next_cache=True)
        _native.profile_enable(True)
        for t in range(n_steps):
            _, cache = model(xs[:, t:t + 1], cache=cache)
        rec = _native.profile_read()
        _native.profile_enable(False)
    stream_ms = [ms for name, ms in rec if name == "decode_stream"]
    finish_ms = [ms for name, ms in rec if name == "decode_finish"]
    n_rec = len(stream_ms)
    # bytes per step: `moved` is what this kernel reads and writes (lookahead keys written back on every 4th
    # step, 16 bytes of cached gates per row read while tokens are pending, 4 written per row otherwise);
    # `reference` is what the reference's step moves (every lookahead key rewritten on every step):
    # B*H*(5*t*d + 8*d)*2.  The roofline figures use the bytes moved.
    bytes_moved = sum(decode_step_bytes(B, H, prefill + i, d, 2, prefill) for i in range(n_rec))
    bytes_reference = sum(B * H * (5 * (prefill + i) * d + 8 * d) * 2 for i in range(n_rec))
    kern_s = (sum(stream_ms) + sum(finish_ms)) * 1e-3
    gbs = bytes_moved / (sum(stream_ms) * 1e-3) / 1e9
    out["kernel_ms_per_step"] = round(kern_s * 1e3 / max(1, n_rec), 4)
    out["kernel_tokens_per_s"] = round(B * n_rec / kern_s, 1)
    rec = recorded_traffic()
    out["roofline"] = {"bound": "hbm", "kernel": "decode_stream", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                       "bytes_per_step": round(bytes_moved / max(1, n_rec)),
                       "traffic": rec.get("bytes", {}).get("decode_stream"), "traffic_source": rec.get("source"),
                       "reference_bytes_per_step": round(bytes_reference / max(1, n_rec)),
                       "reference_bytes_GBps": round(bytes_reference / (sum(stream_ms) * 1e-3) / 1e9, 1)}
    # the whole step (two projections, stream and finish kernels) against the bytes moved
    out["end_to_end_GBps"] = round(bytes_moved / (t2 - t1) / 1e9 * (n_rec / n_steps), 1)
    out["end_to_end_frac_of_hbm_peak"] = round(out["end_to_end_GBps"] / PEAK_HBM_GBS, 4)
    out["workload"] = f"config 4: B{B} H{H} d{d} bf16, prefill {prefill}, {n_steps} cached steps"
    for k in ("prefill_tokens_per_s", "tokens_per_s", "ms_per_decode_step"):
        out[k] = round(out[k], 3)
    return out


def bench_lm(steps=5, warmup=2):
    import torch

    from lookahead_keys_attention_amd import CastleLM

    dev = torch.device("cuda:0")
    B, n, depth, dim, H, d = 16, 1024, 12, 512, 8, 64
    torch.manual_seed(0)
    model = CastleLM(num_tokens=256, dim=dim, depth=depth, heads=H, dim_head=d, use_triton=True,
                     tie_embedding=True).to(dev).bfloat16()
    x = torch.randint(0, 256, (B, n + 1), generator=torch.Generator().manual_seed(0)).to(dev)

    def step():
        model.zero_grad(set_to_none=True)
        model(x, return_loss=True).backward()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    core = 19.0 * B * H * float(n) * n * d * depth
    # generation: 16 prompts of 512 tokens, 128 new tokens each, every layer on its own cache.  The
    # token steps are replays of one captured HIP graph (captured by the warm-up call, kept by the
    # model); the timed call covers prefill, loading the caches into the graph's buffers, 127
    # replays and the sampling between them.  The step-by-step path is timed beside it.
    prompt = x[:, :512]
    model.eval()
    model.sample(prompt, 512 + 16, temperature=1.0)   # also loads the sampling kernels
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.sample(prompt, 512 + 128, temperature=1.0)
    torch.cuda.synchronize()
    gen_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    model.sample(prompt, 512 + 128, temperature=1.0, graph=False)
    torch.cuda.synchronize()
    eager_s = time.perf_counter() - t0
    return {"workload": "config 5: 12 x [Castle(512, 8 heads, 64) + MLP], tied embedding, rotary, prenorm, tokens (16, 1024), bf16",
            "ms_per_step": round(ms, 3), "tokens_per_s": round(B * n / (ms * 1e-3), 1),
            "attention_core_tflops_lower_bound": round(core / (ms * 1e-3) / 1e12, 2),
            "generate_tokens_per_s": round(B * 128 / gen_s, 1),
            "generate_tokens_per_s_without_graph": round(B * 128 / eager_s, 1),
            "generate": "16 prompts x 512 tokens pre-filled, 128 sampled tokens each (top-k 0.9, temperature 1); "
                        "token steps replayed from one captured HIP graph"}


def cpu_baseline(budget_s=20.0):
    """Dense oracle (fp32, autograd backward) on single heads of config 2, as many as fit the budget."""
    import torch

    from oracle import castle_oracle as O

    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    L, d = 4096, 64
    g = torch.Generator().manual_seed(0)
    done, t_used = 0, 0.0
    while done < 32 and (done == 0 or t_used + t_used / done < budget_s):
        ops = [(torch.randn(L, d, generator=g) * 0.6).requires_grad_() for _ in range(6)]
        do = torch.randn(L, d, generator=g)
        t0 = time.perf_counter()
        out = O.parallel_core(*ops, d ** -0.5)
        out.backward(do)
        t_used += time.perf_counter() - t0
        done += 1
    flop = 19.0 * L * L * d * done
    return {"value": round(flop / t_used / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{done} of 32 (batch, head) slices of config 2, dense fp32 forward + autograd backward, "
                      f"{t_used:.1f} s; same algorithmic flop count (19*L^2*d per slice)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-lm", action="store_true")
    ap.add_argument("--no-long-context", action="store_true",
                    help="skip benchmark configuration 3 (seq 16384, dim_head 128; ~27 GB of workspace)")
    ap.add_argument("--long-context", action="store_true", help="kept for compatibility: configuration 3 runs by default")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy four times (reference for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters to bytes)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from lookahead_keys_attention_amd import _native

    if not _native.is_built():
        from lookahead_keys_attention_amd.build import build

        build()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    layer = bench_layer(args.steps, args.warmup)
    line = {
        "metric": "CASTLE fwd+bwd TFLOP/s (bf16, L=4096)",
        "value": round(layer["value"], 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(layer["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "config 2: one Castle layer forward+backward, dim 512, 8 heads, dim_head 64, "
                               "batch 4, seq 4096, bf16 tensors (fp16 MFMA operands, fp32 accumulation)",
                   "global_batch": layer["global_batch"], "seq_len": layer["seq_len"], "parallelism": "single GPU"},
        "core": layer["core"],
        "roofline": layer["roofline"],
    }
    if not args.no_decode:
        line["decode"] = bench_decode()
    if not args.no_lm:
        line["lm"] = bench_lm()
    if not args.no_long_context:
        line["long_context"] = bench_long_context()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
