#!/usr/bin/env python3
"""Benchmark of the XAttention prefill path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 2]

A step is one pass of the hot path - antidiagonal estimate, block selection,
block-sparse attention - over one synthetic single-layer workload whose q/k/v
already sit in HBM.  The default workload is the headline one (L=131072,
32 query / 8 KV heads, d=128, stride 16, tau 0.9, chunk 16384, causal, bf16).
Prints ONE JSON line: the per-layer time (estimate + sparse), the speedup over
this library's own dense causal FlashAttention, the roofline of the dominant
kernel (block-sparse attention, bf16 MFMA, flops of the computed blocks) and a
CPU baseline (the torch restatement of the reference path on workload 0).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "x-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per launch come from the FETCH_SIZE / WRITE_SIZE counter runs (counters cannot be read from inside
# this process): the summary of those runs for the headline workload is kept as a table under profiles/ and read here.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "bench_headline_hbm_traffic.md")
HEADLINE = "cfg2_llama8b_L131072_gqa32x8_S16"


def measured_traffic_bytes(kernel_prefix):
    """Scaled total bytes of the first table row of the traffic summary whose kernel name starts with
    ``kernel_prefix`` (last column, in GB), or None when the summary or the row is missing."""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
                if len(cells) >= 6 and cells[0].startswith(kernel_prefix):
                    return float(cells[-1]) * 1e9
    except (OSError, ValueError):
        pass
    return None


def _ms(a, b):
    return a.elapsed_time(b)


def cpu_baseline(reps=5, warmup=2):
    """Times the oracle (torch restatement of the reference's torch path) on the
    host cores: workload 0 exactly (fp32, L=4096, 32 heads, stride 8, chunk 2048)."""
    import torch

    from oracle import xattn_oracle as O
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[0]
    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)
    q, k, v = make_inputs(w, device="cpu", seed=0)
    t_est, t_att = [], []
    mask = None
    with torch.no_grad():
        for i in range(warmup + reps):
            t0 = time.perf_counter()
            _, mask = O.xattn_estimate(q, k, 128, w.stride, threshold=w.threshold, chunk_size=w.chunk_size, causal=True)
            t1 = time.perf_counter()
            O.block_sparse_attention(q, k, v, mask, causal=True)
            t2 = time.perf_counter()
            if i >= warmup:
                t_est.append((t1 - t0) * 1e3)
                t_att.append((t2 - t1) * 1e3)
    est, att = statistics.median(t_est), statistics.median(t_att)
    with torch.no_grad():
        # the other setting of the torch-branch slice quirk (keys of earlier chunks visible), for the record
        _, mask_all_keys = O.xattn_estimate(q, k, 128, w.stride, threshold=w.threshold, chunk_size=w.chunk_size,
                                            causal=True, pad0_quirk=False)
        torch.set_num_threads(1)
        t0 = time.perf_counter()
        _, m1 = O.xattn_estimate(q, k, 128, w.stride, threshold=w.threshold, chunk_size=w.chunk_size, causal=True)
        O.block_sparse_attention(q, k, v, m1, causal=True)
        single = (time.perf_counter() - t0) * 1e3
        torch.set_num_threads(threads)
    with torch.no_grad():
        # for the GPU-vs-oracle mask comparison below: the oracle on the very bf16 values the GPU path reads
        qb, kb = q.bfloat16().float(), k.bfloat16().float()
        bf16_sums, bf16_mask = O.xattn_estimate(qb, kb, 128, w.stride, threshold=w.threshold, chunk_size=w.chunk_size,
                                                causal=True)
    return {
        "value": round(est + att, 3),
        "unit": "ms per layer",
        "cores": threads,
        "kind": "port",
        "sample": (
            "workload 0 (fp32, L=4096, 32 heads, stride 8, tau 0.9, chunk 2048, causal): oracle xattn_estimate "
            f"+ dense masked softmax attention, median of {reps} after {warmup} warm-ups; the headline L=131072 "
            "does not finish on a CPU in bounded time"
        ),
        "estimate_ms": round(est, 3),
        "attention_ms": round(att, 3),
        "torch_threads": torch.get_num_threads(),
        "os_cpu_count": cores,
        "torch": torch.__version__,
        "single_thread_ms": round(single, 1),
        "mask_density": round(float(mask.float().mean()), 4),
        "mask_density_all_earlier_keys_visible": round(float(mask_all_keys.float().mean()), 4),
    }, (q, k, v, bf16_sums, bf16_mask)


def decode_leg(q, k, v, reps=50):
    """One decode step (the token after the prefill) over the workload's KV cache.

    Not part of the headline value: its own object on the line, with the HBM
    roofline that bounds it (the step reads K and V once: 2 * H_kv * L * 256 bytes).
    """
    import torch
    from xattn.src import hip_backend
    from xattn.src.decode import single_decode_with_kv_cache

    lib = hip_backend.lib()
    heads, kv_heads, L = q.shape[1], k.shape[1], k.shape[2]
    q1 = q[0, :, -1].contiguous()
    ws = torch.empty(lib.xattn_decode_workspace_bytes(heads, kv_heads, L), dtype=torch.uint8, device=q.device)
    out = torch.empty(heads, 128, dtype=q.dtype, device=q.device)
    for _ in range(5):
        single_decode_with_kv_cache(q1, k[0], v[0], kv_layout="HND", out=out, workspace=ws)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        single_decode_with_kv_cache(q1, k[0], v[0], kv_layout="HND", out=out, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    us = _ms(e0, e1) * 1e3 / reps
    nbytes = 2.0 * kv_heads * L * 256
    tbs = nbytes / (us * 1e-6) / 1e12
    return {
        "kernels": "decode_partial_kernel + decode_merge_kernel",
        "kv_len": L, "us_per_step": round(us, 1), "bytes": nbytes,
        "roofline": {"bound": "hbm", "achieved": round(tbs * 1e3, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(tbs * 1e3 / PEAK_HBM_GBS, 4)},
    }


def mfma_probe(dev):
    """What a stream of bf16 MFMAs sustains on this part: alone, and with the vector-ALU load of an attention
    tile (one exponential and three fmas per MFMA, no dependences, no memory) issued beside it; each with constant
    operand bits and with random ones (the clock the part holds depends on the switching activity of the operands)."""
    import ctypes

    import torch
    from xattn.src import hip_backend

    lib = hip_backend.lib()
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    res = {}
    gen = torch.Generator(device="cpu").manual_seed(0)
    tables = {
        "constant_operands": torch.full((4096 * 8,), 0.5, dtype=torch.bfloat16),
        "random_operands": torch.randn(4096 * 8, generator=gen).bfloat16(),
    }
    for name, host in tables.items():
        bits = host.to(dev)
        for mix, suffix in ((0, ""), (1, "_with_softmax_valu_mix")):
            flops = ctypes.c_double(0.0)
            stream = torch.cuda.current_stream().cuda_stream
            hip_backend.check(lib.xattn_mfma_rate_probe(bits.data_ptr(), 20000, mix, sink.data_ptr(), ctypes.byref(flops), stream), "probe")
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            hip_backend.check(lib.xattn_mfma_rate_probe(bits.data_ptr(), 100000, mix, sink.data_ptr(), ctypes.byref(flops), stream), "probe")
            e1.record()
            torch.cuda.synchronize()
            res[name + suffix + "_tflops"] = round(flops.value / (_ms(e0, e1) * 1e-3) / 1e12, 1)
    return res


def density_sweep(w, L, chunk, dev, t_dense, qkv, steps=3):
    """The headline shape at other operating points, so that estimate share and speedup are read against a range
    of densities: thresholds 0.9 / 0.95 / 0.99 on the workload's inputs, and the per-token reading of the rank-8
    term (diffuse attention) at 0.9.  Same timing protocol as the headline, fewer steps."""
    import torch
    from xattn.src.Xattention import block_sparse_attention, estimate_and_select
    from xattn.synthetic import make_inputs

    rows = []
    nb = (L + 127) // 128
    full_blocks = w.heads * nb * (nb + 1) // 2
    n_r = ((L + chunk - 1) // chunk * chunk) // w.stride
    f_est = 2.0 * w.stride * 128 * w.heads * n_r * (n_r + 1) / 2
    for rank8, taus in (("head", (0.9, 0.95, 0.99)), ("token", (0.9,))):
        q, k, v = qkv if rank8 == "head" else make_inputs(w, device=dev, seed=0, L=L, dtype=torch.bfloat16, rank8=rank8)
        for tau in taus:
            for i in range(steps + 1):
                marks = []
                r = estimate_and_select(q, k, w.stride, tau, chunk, causal=True, marks=marks, want_mask=False)
                block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], causal=True)
                end = torch.cuda.Event(enable_timing=True)
                end.record()
                torch.cuda.synchronize()
                m = dict(marks)
                if i == 0:
                    acc = [0.0, 0.0, 0.0]
                    continue
                acc[0] += _ms(m["estimate_begin"], m["select_begin"]) / steps
                acc[1] += _ms(m["select_begin"], m["select_end"]) / steps
                acc[2] += _ms(m["select_end"], end) / steps
            n_sel = int(r["col_cnt"][:, :nb].sum().item())
            total = sum(acc)
            rows.append({
                "rank8": rank8, "threshold": tau, "density": round(n_sel / full_blocks, 4),
                "estimate_ms": round(acc[0], 3), "select_ms": round(acc[1], 3), "sparse_attn_ms": round(acc[2], 3),
                "total_ms": round(total, 3), "estimate_share": round((acc[0] + acc[1]) / total, 4),
                "estimate_pflops": round(f_est / (acc[0] * 1e-3) / 1e15, 3),
                "sparse_pflops": round(4.0 * 128 ** 3 * n_sel / (acc[2] * 1e-3) / 1e15, 3),
                "speedup_vs_dense_fa": round(t_dense / total, 2),
            })
        del q, k, v
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", type=int, default=2, help="index into the synthetic workloads (default: headline)")
    ap.add_argument("--dense-steps", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode-step measurement")
    ap.add_argument("--no-mfma-probe", action="store_true", help="skip the MFMA-only rate probe")
    ap.add_argument("--compare-pipelined", action="store_true",
                    help="also time Xattention_prefill with and without chunk-by-chunk stream pipelining")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (reads 1 GiB, writes 1 GiB) so that HBM byte "
                         "counters collected over this command can be scaled by a kernel of known traffic")
    ap.add_argument("--seq-len", type=int, default=None, help="override L (debug only; invalidates the metric)")
    ap.add_argument("--threshold", type=float, default=None,
                    help="override the workload's tau (a point of the density sweep; the headline value uses the workload's own)")
    ap.add_argument("--rank8", choices=("head", "token"), default="head",
                    help="reading of the text workloads' shared rank-8 component (see xattn/synthetic.py)")
    ap.add_argument("--no-density-sweep", action="store_true",
                    help="skip the extra timings of the headline shape at other thresholds / the per-token generator")
    ap.add_argument("--no-mask-parity", action="store_true", help="skip the oracle run on two heads of the workload")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the prefill path uses no collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from xattn.src import hip_backend
    from xattn.src.Xattention import block_sparse_attention, default_chunk_size, estimate_and_select
    from xattn.synthetic import WORKLOADS, make_inputs

    hip_backend.lib()   # fail loudly if the HIP library has not been built
    if not torch.cuda.is_available():
        raise SystemExit("no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = WORKLOADS[args.workload]
    L = args.seq_len or w.L
    tau = w.threshold if args.threshold is None else args.threshold
    q, k, v = make_inputs(w, device=dev, seed=0, L=L, dtype=torch.bfloat16, rank8=args.rank8)
    chunk = w.chunk_size or default_chunk_size(L)
    torch.cuda.synchronize()

    def step(marks=None):
        # what the operator itself runs: column lists only, no byte mask
        r = estimate_and_select(q, k, w.stride, tau, chunk, causal=w.causal, marks=marks, want_mask=False)
        if marks is not None:
            marks.append(("sparse_begin", marks[-1][1]))
        out = block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], causal=w.causal)
        if marks is not None:
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            marks.append(("sparse_end", ev))
        return r, out

    with torch.no_grad():
        for _ in range(args.warmup):
            r, out = step()
        torch.cuda.synchronize()
        all_marks = []
        t0 = time.perf_counter()
        for _ in range(args.steps):
            m = []
            r, out = step(m)
            all_marks.append(dict(m))
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

        t_est = statistics.mean(_ms(m["estimate_begin"], m["select_begin"]) for m in all_marks)
        t_sel = statistics.mean(_ms(m["select_begin"], m["select_end"]) for m in all_marks)
        t_sparse = statistics.mean(_ms(m["sparse_begin"], m["sparse_end"]) for m in all_marks)
        t_total = statistics.mean(_ms(m["estimate_begin"], m["sparse_end"]) for m in all_marks)

        # dense causal FlashAttention written the same way (same kernel, every visible block)
        block_sparse_attention(q, k, v, causal=w.causal)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.dense_steps):
            dense = block_sparse_attention(q, k, v, causal=w.causal)
        e1.record()
        torch.cuda.synchronize()
        t_dense = _ms(e0, e1) / args.dense_steps

    nb = (L + 127) // 128
    n_sel = int(r["col_cnt"][:, :nb].sum().item())
    H = w.heads
    full_blocks = H * nb * (nb + 1) // 2 if w.causal else H * nb * nb
    sparsity = 1.0 - n_sel / full_blocks
    f_sparse = 4.0 * 128 * 128 * 128 * n_sel
    f_dense = (4.0 * 128 * H * L * (L + 1) / 2) if w.causal else (4.0 * 128 * H * L * L)
    n_r = ((L + chunk - 1) // chunk * chunk) // w.stride
    f_est = (2.0 * w.stride * 128 * H * n_r * (n_r + 1) / 2) if w.causal else (2.0 * w.stride * 128 * H * n_r * n_r)
    nkb_p = (L + chunk - 1) // chunk * chunk // 128
    sel_bytes = H * nkb_p * nkb_p * 5 + 4 * (n_sel + H * nkb_p)
    sparse_tflops = f_sparse / (t_sparse * 1e-3) / 1e12
    est_tflops = f_est / (t_est * 1e-3) / 1e12
    as_configured = L == w.L and args.threshold is None and args.rank8 == "head"
    headline_traffic = as_configured and w.name == HEADLINE
    roofline_sparse = {
        "kernel": "block_sparse_fwd_kernel<true>", "bound": "mfma", "achieved": round(sparse_tflops, 1),
        "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(sparse_tflops / PEAK_BF16_TFLOPS, 4),
        "ms": round(t_sparse, 3), "flop": f_sparse,
        "traffic": measured_traffic_bytes("xattn::block_sparse_fwd_kernel<true>") if headline_traffic else None,
    }
    # the estimator stage is one entry point = the MFMA kernel plus its short normalisation pass (about 6 % of the
    # stage at the headline); its time is taken between the same stream events
    roofline_est = {
        "kernel": "estimate_gemm_kernel (+ estimate_normalize_kernel, same entry point)", "bound": "mfma",
        "achieved": round(est_tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
        "frac": round(est_tflops / PEAK_BF16_TFLOPS, 4), "ms": round(t_est, 3), "flop": f_est,
        "traffic": measured_traffic_bytes("xattn::estimate_gemm_kernel") if headline_traffic else None,
    }
    dominant = roofline_est if t_est >= t_sparse else roofline_sparse

    result = {
        "metric": "per-layer prefill attn ms (estimate+sparse) at 128k; speedup vs dense FA",
        "value": round(t_total, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": (w.name if L == w.L else f"{w.name}@L={L}") + ("" if args.rank8 == "head" else "@rank8=token"),
            "seq_len": L, "q_heads": H, "kv_heads": w.kv_heads, "head_dim": 128, "stride": w.stride,
            "threshold": tau, "chunk_size": chunk, "block_size": 128, "causal": w.causal,
            "estimator_semantics": "all earlier keys visible (reference Triton branch)",
        },
        "estimate_ms": round(t_est, 3),
        "select_ms": round(t_sel, 3),
        "sparse_attn_ms": round(t_sparse, 3),
        "dense_fa_ms": round(t_dense, 3),
        "speedup_vs_dense_fa": round(t_dense / t_total, 3),
        "estimate_fraction_of_total": round((t_est + t_sel) / t_total, 4),
        "sparsity": round(sparsity, 4),
        "selected_blocks": n_sel,
        "estimate_tflops": round(est_tflops, 1),
        "dense_fa_tflops": round(f_dense / (t_dense * 1e-3) / 1e12, 1),
        "select_gbs": round(sel_bytes / (t_sel * 1e-3) / 1e9, 1),
        # the launch that takes longest of the two MFMA stages; both are listed after it
        "roofline": dict(dominant),
        "roofline_estimator": roofline_est,
        "roofline_sparse_attention": roofline_sparse,
    }
    del dense, out
    if not args.no_mask_parity and w.causal is not None:
        # block-mask parity with the oracle (fp32, on the same bf16 values) for the query heads with the fewest and
        # the most kept blocks: mismatches, and how many of them the contract allows (within 1e-5 of tau, or runs of
        # equal sums cut by the crossing)
        from oracle.parity import head_mask_parity

        kept = r["col_cnt"].long().sum(-1)
        heads = sorted({int(kept.argmin()), int(kept.argmax())})
        r = estimate_and_select(q, k, w.stride, tau, chunk, causal=w.causal, want_lists=False)     # with the mask
        tot = {"blocks": 0, "mismatches": 0, "in_band": 0, "ties": 0, "outside_band": 0}
        for h in heads:
            rep = head_mask_parity(q, k, h, r["mask"][h], w.stride, tau, chunk, w.causal, pad0_quirk=False)
            for key in tot:
                tot[key] += rep[key]
        tot["heads"] = heads
        result["mask_parity"] = tot
    if (not args.no_density_sweep) and as_configured and w.name == HEADLINE:
        result["density_sweep"] = density_sweep(w, L, chunk, dev, t_dense, (q, k, v))
    if args.compare_pipelined:
        from xattn.src.Xattention import Xattention_prefill

        for flag in (False, True):
            for _ in range(2):
                Xattention_prefill(q, k, v, w.stride, threshold=w.threshold, chunk_size=chunk, causal=w.causal,
                                   pipeline_chunks=flag)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                Xattention_prefill(q, k, v, w.stride, threshold=w.threshold, chunk_size=chunk, causal=w.causal,
                                   pipeline_chunks=flag)
            e1.record()
            torch.cuda.synchronize()
            result["operator_ms_pipelined" if flag else "operator_ms_single_launch"] = round(_ms(e0, e1) / args.steps, 3)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        hip_backend.check(
            hip_backend.lib().xattn_calibration_copy(
                dst.data_ptr(), src.data_ptr(), src.numel() * 4, torch.cuda.current_stream().cuda_stream
            ),
            "xattn_calibration_copy",
        )
        torch.cuda.synchronize()
        del src, dst
    if not args.no_decode:
        result["decode_step"] = decode_leg(q, k, v)
    if not args.no_mfma_probe:
        result["mfma_alone"] = mfma_probe(dev)
    if not args.no_cpu_baseline:
        base, (cq, ck, cv, csums, cmask) = cpu_baseline()
        # the same sample on the GPU path (bf16), for scale
        gq, gk, gv = cq.to(dev).bfloat16(), ck.to(dev).bfloat16(), cv.to(dev).bfloat16()
        w0 = WORKLOADS[0]
        for _ in range(3):
            rr = estimate_and_select(gq, gk, w0.stride, w0.threshold, w0.chunk_size, causal=True, use_triton=False)
            block_sparse_attention(gq, gk, gv, rr["col_idx"], rr["col_cnt"], causal=True)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            rr = estimate_and_select(gq, gk, w0.stride, w0.threshold, w0.chunk_size, causal=True, use_triton=False)
            block_sparse_attention(gq, gk, gv, rr["col_idx"], rr["col_cnt"], causal=True)
        e1.record()
        torch.cuda.synchronize()
        base["gpu_same_sample_ms"] = round(_ms(e0, e1) / 10, 3)
        # GPU mask against the oracle's on identical values (the sample rounded to bf16, oracle in fp32)
        from oracle.parity import mask_mismatch_detail

        d = mask_mismatch_detail(csums[0], rr["mask"], cmask[0], w0.threshold, True, 0, w0.chunk_size // 128)
        base["gpu_mask_vs_oracle_same_inputs"] = {"blocks": int(cmask[0].numel()), **d}
        result["cpu_baseline"] = base
    print(json.dumps(result))


if __name__ == "__main__":
    main()
