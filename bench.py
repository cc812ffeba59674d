"""Benchmark of the VQ-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one seqlen_q = 1 VQ-attention call (lookup table + streaming kernel; a split merge where a (batch, head)
unit is split, which this workload is not) over the decode
configuration: batch 16, 32 heads, head_dim 128, 32768 keys, 4 codebooks x 256 codewords, bf16, inputs resident in
HBM.  Prints ONE JSON line.  `value` is the achieved HBM rate of the whole step: algorithmic bytes (codes + V +
codebooks + q + out, each touched once) divided by the step time.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# HBM bytes one launch of the streaming kernel moves at the default workload: a counter measurement (rocprofv3
# FETCH_SIZE / WRITE_SIZE scaled by a 1 GiB copy in the same run), not something this script can observe; the figure
# and the file that documents the run that produced it travel together
DECODE_MAIN_KERNEL_TRAFFIC = {
    "bytes": 4_364_264_000,
    "source": "profiles/decode_main_kernel_c2_b16_h32_n32768.md (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE; "
              "not measured by this run)",
}


def cpu_baseline(case, units=256, repeats=5):
    """The fp32 PyTorch oracle timed on the host cores over `units` (batch, head) problems of the same workload.

    Returns the equivalent HBM rate (algorithmic bytes of the sampled units / time) so it is comparable with `value`.
    """
    import torch

    import oracle

    B, H = case.q.shape[:2]
    units = min(units, B * H)
    idx = [(u * 7) % (B * H) for u in range(units)]  # spread over batches and heads
    sample = []
    for u in idx:
        b, h = divmod(u, H)
        sample.append((case.q[b:b + 1, h:h + 1].cpu(), case.codes[b:b + 1, h:h + 1].cpu(),
                       case.codebooks[h:h + 1].cpu(), case.v[b:b + 1, h:h + 1].cpu()))
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    times = []
    for r in range(repeats + 1):
        t0 = time.perf_counter()
        for q, c, cb, v in sample:
            oracle.attn_vq_decode(q, c, cb, v, case.softmax_scale)
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[len(times[1:]) // 2]
    e = case.q.element_size()
    D = case.q.shape[-1]
    N, M = case.codes.shape[2], case.codes.shape[3]
    bytes_per_unit = N * M + N * D * e + case.codebooks[0].numel() * e + 2 * D * e
    return {
        "value": round(units * bytes_per_unit / t / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{units} of {B * H} (batch, head) units of the same workload, fp32 PyTorch oracle, "
                  f"median of {repeats} runs, {t * 1e3:.1f} ms",
    }


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def _cpu_time(fn, repeats=3):
    import torch

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], cores


def _time_events(fn, steps, warmup):
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    # median: after an idle period (tensor set-up, the CPU baseline) a compute-bound kernel first slows down by ~10 %
    # over half a dozen calls and then speeds up for another fifty (a 0.6 ms kernel: 660 -> 745 -> 555 us over 60
    # consecutive calls; clock / power management), hence also the long warm-ups below
    ms = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))
    return ms[len(ms) // 2]


def prefill_extra(dev, steps=60, warmup=60, cpu=True):
    """Second half of the metric: causal VQ-attention prefill at 8k with a 1024-key exact window (not part of the
    timed decode region).  Reported as algorithmic TFLOP/s and as a fraction of the bf16 MFMA peak."""
    import torch

    from vqtree_amd.ops.attn_vq import attn_vq_prefill
    from vqtree_amd.synthetic import prefill_c3

    case = prefill_c3(dev)
    fn = lambda: attn_vq_prefill(case.q, case.codes, case.codebooks, case.v, k_exact=case.k_exact,
                                 window_size=case.window, softmax_scale=case.softmax_scale)
    ms = _time_events(fn, steps, warmup)
    flops = case.algorithmic_flops("block")
    B, H, N, D = case.q.shape
    tf = flops / (ms * 1e-3) / 1e12
    out = {
        "workload": f"causal VQ-attention prefill: batch {B}, {H} heads, head_dim {D}, seq {N}, exact window "
                    f"{case.window} (block boundary rule), {case.codes.shape[3]} codebooks x "
                    f"{case.codebooks.shape[2]}, bf16",
        "us_per_call": round(ms * 1e3, 1),
        "algorithmic_gflop": round(flops / 1e9, 2),
        "tflops": round(tf, 1),
        "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "duration_covers": "whole call: key reconstruction kernel + fused window/far attention kernel",
                     # attention kernel 356.3 MB fetched + 67.1 MB written, reconstruction 66.0 MB fetched + 57.7 written
                     "traffic": 356_322_000 + 67_109_000 + 66_003_000 + 57_676_000,
                     "traffic_source": "profiles/prefill_pipe_kernel_vq_prefill_c3_h32_n8192_w1024.md (rocprofv3 --pmc "
                                       "FETCH_SIZE, then WRITE_SIZE; not measured by this run)"},
    }
    if cpu:
        # the oracle on one of the H independent heads (same inputs), rate extrapolated over heads
        import oracle

        h = 0
        args = [x[:, h:h + 1].cpu() for x in (case.q, case.codes)] + [case.codebooks[h:h + 1].cpu(), case.v[:, h:h + 1].cpu()]
        k_ex = case.k_exact[:, h:h + 1].cpu()
        t, cores = _cpu_time(lambda: oracle.attn_vq_prefill(*args, k_exact=k_ex, window_size=case.window,
                                                            softmax_scale=case.softmax_scale), repeats=3)
        out["cpu_baseline"] = {
            "value": round(flops / (B * H) / t / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"1 of {B * H} (batch, head) units of the same workload (heads are independent, rate "
                      f"extrapolated), fp32 PyTorch oracle, median of 3 runs, {t * 1e3:.0f} ms",
        }
    del case
    torch.cuda.empty_cache()
    return out


def local_rerope_extra(dev, steps=60, warmup=60, cpu=True):
    """Sliding-window ReRoPE attention at 16k (batch 2, 32 heads, window 512), the exact-window building block of the
    prefill path: useful FLOPs = 4 * D * visible pairs (keys j <= i with j >= floor(i/128)*128 - window)."""
    import torch

    from vqtree_amd.ops.attn_vq import rope_tables, rotate_half
    from vqtree_amd.ops.triton_fused_local_attn_rerope import flash_attn_func

    B, H, N, D, W = 2, 32, 16384, 128, 512
    g = torch.Generator(device=dev).manual_seed(4)
    q, k, v = (torch.randn(B, N, H, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    cos, sin = rope_tables(D, N, dtype=torch.bfloat16, device=dev)
    rope = lambda x, c, s_: x * c + rotate_half(x) * s_
    q1, k1 = rope(q, cos[None, :, None], sin[None, :, None]), rope(k, cos[None, :, None], sin[None, :, None])
    q2 = rope(q, cos[W + 1], sin[W + 1])
    ms = _time_events(lambda: flash_attn_func(q1, q2, k1, k, v, W), steps, warmup)
    i = torch.arange(N, dtype=torch.int64)
    pairs = int((i - torch.clamp(i // 128 * 128 - W, min=0) + 1).sum())
    flops = 4 * D * pairs * B * H
    tf = flops / (ms * 1e-3) / 1e12
    out = {
        "workload": f"local ReRoPE window attention: batch {B}, {H} heads, head_dim {D}, seq {N}, window {W}, bf16",
        "us_per_call": round(ms * 1e3, 1),
        "useful_gflop": round(flops / 1e9, 1),
        "tflops": round(tf, 1),
        "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
        "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "duration_covers": "the one window kernel",
                     "traffic": 1_701_251_000 + 268_443_000,
                     "traffic_source": "profiles/window_pipe_kernel_local_rerope_c4_b2_h32_n16384_w512.md (rocprofv3 --pmc "
                                       "FETCH_SIZE, then WRITE_SIZE; not measured by this run)"},
    }
    if cpu:
        import oracle

        b, h = 0, 0
        args = [x[b:b + 1, :, h:h + 1].transpose(1, 2).cpu() for x in (q1, k1, v)]
        q2c, kc = (x[b:b + 1, :, h:h + 1].transpose(1, 2).cpu() for x in (q2, k))
        t, cores = _cpu_time(lambda: oracle.local_attn(*args, W, "rerope", None, q2=q2c, k2=kc), repeats=3)
        out["cpu_baseline"] = {
            "value": round(flops / (B * H) / t / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"1 of {B * H} (batch, head) units of the same workload (units are independent, rate "
                      f"extrapolated), fp32 PyTorch oracle with dense masks, median of 3 runs, {t * 1e3:.0f} ms",
        }
    del q, k, v, q1, k1, q2
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the (untimed-region) prefill measurement")
    ap.add_argument("--no-c5", action="store_true", help="skip the (untimed-region) 32-layer decode harness")
    ap.add_argument("--c5-steps", type=int, default=128, help="decode steps of the 32-layer harness (the configured 128)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the timed region, run one plain 1 GiB device copy (reference dispatch of known "
                         "size for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU only: the VQ-attention path shards over (batch, head) with no "
                 "communication, and this build runs on single-GPU boxes; run with --gpus 1")

    import torch

    from vqtree_amd import _lib
    from vqtree_amd.ops.attn_vq import attn_vq_decode
    from vqtree_amd.synthetic import decode_c2

    _lib.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    case = decode_c2(dev)
    B, H, N, M = case.codes.shape
    D = case.q.shape[-1]
    K = case.codebooks.shape[2]

    def step():
        return attn_vq_decode(case.q, case.codes, case.codebooks, case.v, softmax_scale=case.softmax_scale)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # HIP events on the stream the kernels run on (torch's current stream is the one handed to the library)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record()
        step()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    ms_per_step = wall * 1e3 / args.steps
    kern_ms = sum(ev_ms) / len(ev_ms)

    alg_bytes = case.algorithmic_bytes
    value = alg_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = alg_bytes / (kern_ms * 1e-3) / 1e9
    result = {
        "metric": "VQ-attn decode HBM GB/s @32k (us/step in us_per_step)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "us_per_step": round(ms_per_step * 1e3, 1),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"VQ-attention decode seqlen_q=1: batch {B}, {H} heads, head_dim {D}, KV context {N}, "
                        f"{M} codebooks x {K} codewords, uint8 codes, bf16 q/V/codebooks, no mask",
            "algorithmic_bytes_per_step": alg_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": DECODE_MAIN_KERNEL_TRAFFIC["bytes"],
            "traffic_source": DECODE_MAIN_KERNEL_TRAFFIC["source"],
            "kernel": "vqa::decode::main_kernel<bf16,128,4>",
            "duration_us": round(kern_ms * 1e3, 1),
            "duration_covers": "HIP events around the whole call (lookup-table kernel + streaming kernel, which with "
                               "one split per (batch, head) stores the result itself); the streaming kernel is 99% "
                               "of it",
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case)
    del case
    torch.cuda.empty_cache()
    if not args.no_c5:
        # configuration 5: 32-layer Llama-2-7B-shaped greedy decode over per-layer VQ key caches at 65536 context
        from vqtree_amd import decode_harness

        c5 = decode_harness.run(steps=args.c5_steps, warmup=4)
        c5["roofline"] = {"bound": "hbm", "achieved": c5["attention_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                          "frac": c5["attention_hbm_frac"],
                          "duration_covers": "HIP events around the attention calls of all 32 layers (lookup table "
                                             "with the clamped rotary of the query, streaming kernel, merge), per decode step, launches "
                                             "queued ahead of the GPU",
                          # streaming kernel 2 187.5 MB per layer (fetch + write counters), table and merge kernels 9.9 MB
                          "traffic": 32 * (2_187_461_000 + 9_932_000),
                          "traffic_source": "profiles/decode_harness_c5_b4_n65536.md (rocprofv3 --pmc FETCH_SIZE, then "
                                            "WRITE_SIZE; not measured by this run)"}
        result["c5"] = c5
    torch.cuda.empty_cache()
    if not args.no_prefill:
        result["prefill"] = prefill_extra(dev, cpu=not args.no_cpu_baseline)
        result["local_rerope"] = local_rerope_extra(dev, cpu=not args.no_cpu_baseline)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
