#!/usr/bin/env python3
"""Benchmark of the TQ4 KV-cache hot path on one MI355X.

Headline (one JSON line on stdout): split-K paged TQ4 decode at the
Llama-3-8B single-layer shape of BASELINE.json configs[2] (32 query heads over
8 KV heads, d=128, batch 32, 4096 tokens of context, 16-token pages, seeded
random block tables, bf16 queries).  A step is one decode call for the whole
batch: query rotation + split-K decode + split reduce and output rotation.
`value` is the algorithmic KV bytes of a step (context tokens x KV heads x 136)
divided by the step time, with a different cache every step so that the 256 MB
last-level cache cannot serve it (the "cold" figure).  The same line carries
the roofline of the dominant kernel, the CPU baseline (the oracle timed on the
host cores) and, under "extra", the standalone compress / decompress figures
of configs[1].

    python bench.py --gpus 1 --steps 50 --warmup 5
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published peak
H_Q, H_KV, D, BS = 32, 8, 128, 16
BATCH, CTX = 32, 4096
EXTRA_ITERS = 20              # timed calls of every leg other than the headline
ROW_BYTES = H_KV * (D + 8)
DOMINANT_KERNEL = "paged_decode_staged_kernel<4,4,bf16,4,false,4,0,false,128>"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def outlier_rows(n, h, d, seed, device, dtype=torch.bfloat16):
    """N(0,1) rows, 4 channels per head scaled x10 (the benchmark's outlier rule)."""
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(n, h, d, generator=g, device=device, dtype=torch.float32)
    gc = torch.Generator(device="cpu").manual_seed(seed)
    for head in range(h):
        ch = torch.randperm(d, generator=gc)[:4].to(device)
        x[:, head, ch] *= 10.0
    return x.to(dtype)


def build_cache(K, book, seed, device):
    """One packed paged cache for the decode workload, filled through the HIP
    compress kernel, with a seeded random block table."""
    cent, bnd, rot = book
    n_tok = BATCH * CTX
    pages_per_seq = CTX // BS
    n_pages = BATCH * pages_per_seq
    k = outlier_rows(n_tok, H_KV, D, seed, device)
    v = outlier_rows(n_tok, H_KV, D, seed + 1, device)
    kp, kn = K.tq4_compress(k, rot, bnd)
    vp, vn = K.tq4_compress(v, rot, bnd)
    del k, v
    row = torch.empty(n_tok, ROW_BYTES, dtype=torch.uint8, device=device)
    o1 = H_KV * (D // 2)
    o2 = o1 + 4 * H_KV
    o3 = o2 + H_KV * (D // 2)
    row[:, :o1] = kp.reshape(n_tok, -1)
    row[:, o1:o2] = kn.reshape(n_tok, H_KV).contiguous().view(torch.uint8)
    row[:, o2:o3] = vp.reshape(n_tok, -1)
    row[:, o3:] = vn.reshape(n_tok, H_KV).contiguous().view(torch.uint8)
    g = torch.Generator(device="cpu").manual_seed(2002 + seed)
    table = torch.randperm(n_pages, generator=g).reshape(BATCH, pages_per_seq).to(torch.int32)
    cache = torch.empty(n_pages, BS, ROW_BYTES, dtype=torch.uint8, device=device)
    t = torch.arange(CTX)
    slots = (table.long()[:, t // BS] * BS + (t % BS)).reshape(-1).to(device)   # token (s, t) -> slot
    cache.view(-1, ROW_BYTES)[slots] = row
    return cache, table.to(device)


def time_events(fn, iters):
    """Median and mean time of a call in ms, from GPU events recorded on the stream the calls are
    launched on (torch's current stream) around every call."""
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(iters):
        fn(i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(iters))
    median = each[iters // 2] if iters % 2 else 0.5 * (each[iters // 2 - 1] + each[iters // 2])
    return median, marks[0].elapsed_time(marks[iters]) / iters


def time_region(fn, iters):
    """Average time of a call in ms from two GPU events, one before the first and one after the last of
    `iters` back-to-back calls on torch's current stream (no event between the calls: an event between
    two launches costs the stream a barrier packet of its own, about 2 us here)."""
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    first.record()
    for i in range(iters):
        fn(i)
    last.record()
    torch.cuda.synchronize()
    return first.elapsed_time(last) / iters


def committed_traffic(kernel):
    """HBM bytes per launch of the dominant kernel as the committed counter summary states them (a line
    `TRAFFIC_BYTES_PER_LAUNCH <kernel> <bytes>` in profiles/paged_decode_hbm_traffic_pmc.txt, written from
    FETCH_SIZE / WRITE_SIZE runs), with where the figure comes from: the file, a hash of its bytes and
    the kernel it names.  The figure is None, and `stale` says why, when the summary names another kernel
    than the one this run times: a committed number is only as fresh as the profile it was read from."""
    import hashlib
    rel = os.path.join("profiles", "paged_decode_hbm_traffic_pmc.txt")
    src = {"file": rel, "sha256_16": None, "kernel_in_file": None, "stale": None}
    try:
        raw = open(os.path.join(ROOT, rel), "rb").read()
    except OSError:
        src["stale"] = "summary file missing"
        return None, src
    src["sha256_16"] = hashlib.sha256(raw).hexdigest()[:16]
    for ln in raw.decode().splitlines():
        parts = ln.split()
        if len(parts) == 3 and parts[0] == "TRAFFIC_BYTES_PER_LAUNCH":
            src["kernel_in_file"] = parts[1]
            if parts[1] == kernel:
                return float(parts[2]), src
    src["stale"] = f"the summary does not cover {kernel}"
    return None, src


def output_ulps(err, want, dtype):
    """|err| in units in the last place of the output dtype at the magnitude of the expected value."""
    mant = 7 if dtype == torch.bfloat16 else 10
    mag = want.abs().clamp_min(2.0 ** -14)
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - mant)
    return (err / ulp).max().item()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline leg")
    ap.add_argument("--skip-extra", action="store_true", help="omit the compress / decompress legs")
    ap.add_argument("--skip-other-shapes", action="store_true",
                    help="omit the legs on shapes that are not BASELINE configs (profiles of the configs alone)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain device copy of one cache (142.6 MB read + 142.6 MB written): the "
                         "reference point for scaling the FETCH_SIZE / WRITE_SIZE counters of a profiler run")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this benchmark runs on exactly one GPU (the path has no collectives); use --gpus 1")
        sys.exit(2)
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(3)

    from flashquant_amd import kernels as K
    from flashquant_amd import load_native
    from oracle import tq_oracle as O

    C = load_native()
    dev = torch.device("cuda:0")
    # the product's own host set-up: codebook solver and seeded rotation of the library
    cent, bnd = C.codebook.solve_lloyd_max(D, 4)
    rot = C.haar_orthogonal(D, 42)
    book = (cent.to(dev), bnd.to(dev), rot.to(dev))
    cent_d, _, rot_d = book
    scale = 1.0 / math.sqrt(D)

    # ---- decode workload -----------------------------------------------------------
    n_caches = 4                      # 4 x 143 MB > 256 MB last-level cache
    caches = [build_cache(K, book, 1100 + 10 * i, dev) for i in range(n_caches)]
    gq = torch.Generator(device="cpu").manual_seed(1002)
    q = torch.randn(BATCH, H_Q, D, generator=gq).to(torch.bfloat16).to(dev)
    lens = torch.full((BATCH,), CTX, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    kv_bytes = BATCH * CTX * ROW_BYTES
    n_splits = C.paged_decode_auto_splits(BATCH, H_KV, BS, CTX // BS)

    def step(i):
        cache, table = caches[i % n_caches]
        K.split_k_paged_decode(q, cache, table, lens, cent_d, cent_d, rot_d, H_KV, D, BS,
                               sm_scale=scale, out=out)

    # Untimed, before the W warm-up steps: a quarter of a second of the same steps.  The GPU's clocks take
    # some tens of milliseconds of work to come up from idle (the first few hundred 40 us steps after a
    # pause run 10-25 % slower than the following ones), which W = 20 steps do not cover.
    t_ramp = time.perf_counter()
    i_ramp = 0
    while time.perf_counter() - t_ramp < 0.25:
        for _ in range(50):
            step(i_ramp)
            i_ramp += 1
        torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # The figure reported: exactly K steps back to back between two GPU events, synchronised on both
    # sides, divided by K (the host-side wall clock around the same loop is reported next to it: it
    # also holds what the host needs to issue a step).
    step_ms = time_region(step, args.steps)
    step_median_ms, step_mean_ms = time_events(step, args.steps)
    warm_ms = time_region(lambda i: step(0), args.steps)

    # ---- dominant kernel alone (the split-K decode), cold ----------------------------
    parts = (torch.empty(BATCH, H_Q, n_splits, D, device=dev), torch.empty(BATCH, H_Q, n_splits, device=dev),
             torch.empty(BATCH, H_Q, n_splits, device=dev))

    def decode_only(i):
        cache, table = caches[i % n_caches]
        # the same launch the step makes: un-rotated query, rotation applied in the kernel's prologue
        C.paged_tq4_decode_partials(q, cache, table, lens, cent_d, cent_d, H_KV, D, BS, scale, n_splits, parts, rot_d)

    for i in range(args.warmup):
        decode_only(i)
    kern_ms = time_region(decode_only, args.steps)         # average launch duration
    _, kern_each_ms = time_events(decode_only, args.steps)
    achieved = kv_bytes / (kern_ms * 1e-3) / 1e9

    extra = {
        "decode_tokens_per_s": BATCH / (step_ms * 1e-3),
        "decode_step_us_cold": step_ms * 1e3,
        "decode_step_us_cold_event_median": step_median_ms * 1e3,
        "decode_step_us_warm": warm_ms * 1e3,
        "decode_step_us_wallclock": wall_ms * 1e3,
        "decode_step_us_cold_mean": step_mean_ms * 1e3,
        "decode_gbps_warm": kv_bytes / (warm_ms * 1e-3) / 1e9,
        "decode_pct_hbm_peak_cold": 100.0 * kv_bytes / (step_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "decode_kernel_us_cold": kern_ms * 1e3,
        "decode_kernel_us_cold_event_per_launch": kern_each_ms * 1e3,
        "num_splits": n_splits,
        "kv_bytes_per_step": kv_bytes,
    }

    if args.copy_probe:
        dst = torch.empty_like(caches[0][0])
        for i in range(4):
            dst.copy_(caches[i % n_caches][0])
        torch.cuda.synchronize()
        del dst

    # ---- CPU baseline: the oracle on the host cores, bounded sample ---------------------
    cpu = None
    check = None
    if not args.skip_cpu:
        cache_h = caches[0][0].cpu()
        table_h = caches[0][1].cpu()
        q_h = q.cpu()
        lens_h = lens.cpu()
        # the GPU's result for the same cache, checked row by row against what the oracle computes
        cache0, table0 = caches[0]
        got = K.split_k_paged_decode(q, cache0, table0, lens, cent_d, cent_d, rot_d, H_KV, D, BS,
                                     sm_scale=scale).float().cpu()
        done, spent, worst, worst_abs = 0, 0.0, 0.0, 0.0
        n_elems, n_flat, worst_ulps = 0, 0, 0.0
        while spent < 10.0 and done < 40 * BATCH:      # about 10 s of CPU work, whole sequences
            s_i = done % BATCH
            t1 = time.perf_counter()
            want = O.split_k_paged_decode(q_h[s_i:s_i + 1], cache_h, table_h[s_i:s_i + 1], lens_h[s_i:s_i + 1],
                                          cent, cent, rot, H_KV, D, BS, sm_scale=scale)
            spent += time.perf_counter() - t1
            done += 1
            # 2e-2 of a row's magnitude, never less than 2e-2 absolute: the outlier channels take some
            # output rows beyond |x| = 4, where a single bfloat16 step is 0.03
            w_f = want[0].float()
            row_scale = w_f.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
            worst = max(worst, ((got[s_i] - w_f).abs() / row_scale).max().item())
            worst_abs = max(worst_abs, (got[s_i] - w_f).abs().max().item())
            if done <= BATCH:
                err = (got[s_i] - w_f).abs()
                n_elems += err.numel()
                n_flat += int((err <= 2e-2).sum().item())
                worst_ulps = max(worst_ulps, output_ulps(err, w_f, q.dtype))
        # the reference's CPU fallback as written, a Python loop over tokens and heads, at a reduced shape
        lb, ll = 2, 512
        lens_l = torch.full((lb,), ll, dtype=torch.int32)
        t1 = time.perf_counter()
        want_l = O.paged_decode_loop(torch.matmul(q_h[:lb].float(), rot.T).to(q_h.dtype), cache_h, table_h[:lb], lens_l,
                                     cent, cent, H_KV, D, BS, sm_scale=scale)
        loop_s = time.perf_counter() - t1
        # rotated-space output of a pre-rotated query: what the loop form of the reference returns
        q_rot_d = torch.matmul(q[:lb].float(), rot_d.T).to(q.dtype)
        got_l = C.fused_paged_tq4_decode(q_rot_d, cache0, table0[:lb].contiguous(), lens_l.to(dev), cent_d, cent_d,
                                         None, H_KV, D, BS, sm_scale=scale).float().cpu()
        worst_l = (got_l - want_l.float()).abs().max().item()
        cpu = {
            "value": done * CTX * ROW_BYTES / spent / 1e9,
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{done} sequence decodes ({done / BATCH:.1f} batches) of the same workload with the oracle "
                      f"(vectorised-gather form of the reference's CPU fallback), {spent:.1f} s",
            "loop_form": {
                "value": lb * ll * ROW_BYTES / loop_s / 1e9,
                "unit": "GB/s",
                "sample": f"the reference's token-by-token Python loop at batch {lb} x {ll} tokens, {loop_s:.1f} s",
            },
        }
        check = {
            "max_err_of_row_magnitude": worst, "max_abs_err": worst_abs, "sequences_checked": min(done, BATCH),
            "tolerance": "2e-2 of the row's largest |x|, at least 2e-2 absolute",
            # the same errors read without the scaling: the share of the output elements within a flat
            # 2e-2, and the largest error in units in the last place of the bfloat16 output
            "share_within_flat_2e-2": n_flat / max(n_elems, 1),
            "max_err_ulps_of_output_dtype": worst_ulps,
            "loop_form_max_abs_err": worst_l, "ok": bool(worst <= 2e-2 and worst_l <= 2e-2),
        }
        del cache_h

    # ---- standalone compress / decompress (configs[1]) -----------------------------------
    if not args.skip_extra:
        # a serving decode step as the attention implementation runs it (src/flashquant/vllm/impl.py:220-263,
        # 362-394): the new token's K and V of every sequence are compressed into their cache rows, then the
        # decode runs over the context (here the new token takes the last position of the same contexts)
        ev_s, od_s = C.split_rotation(rot)
        ev_s, od_s = ev_s.to(dev), od_s.to(dev)
        k_new = torch.randn(BATCH, H_KV, D, device=dev).to(torch.bfloat16)
        v_new = torch.randn(BATCH, H_KV, D, device=dev).to(torch.bfloat16)
        last_slots = [(t.long()[:, (CTX - 1) // BS] * BS + (CTX - 1) % BS).contiguous() for _, t in caches]

        def serving_step(i):
            cache, table = caches[i % n_caches]
            K.tq4_compress_and_store(k_new, v_new, rot_d, book[1], cache, last_slots[i % n_caches],
                                     rotation_T_even=ev_s, rotation_T_odd=od_s)
            K.split_k_paged_decode(q, cache, table, lens, cent_d, cent_d, rot_d, H_KV, D, BS, sm_scale=scale, out=out)

        bnd_d = book[1].to(dev)

        def serving_step_one_call(i):
            # the same step through the entry point that stores the new token inside the decode launch
            cache, table = caches[i % n_caches]
            K.tq4_store_and_decode(k_new, v_new, last_slots[i % n_caches], q, cache, table, lens, cent_d, cent_d, rot_d,
                                   bnd_d, H_KV, D, BS, sm_scale=scale, out=out, rotation_T_even=ev_s, rotation_T_odd=od_s)

        for i in range(args.warmup):
            serving_step(i)
        serve2_ms = time_region(serving_step, args.steps)
        for i in range(args.warmup):
            serving_step_one_call(i)
        serve_ms = time_region(serving_step_one_call, args.steps)
        extra.update({"serving_step_us_cold": serve_ms * 1e3, "serving_tokens_per_s": BATCH / (serve_ms * 1e-3),
                      "serving_step_us_cold_store_then_decode": serve2_ms * 1e3})
        # the two forms of the step on one cache: same output (the stored indices may differ where a rotated
        # coordinate lies within float32 rounding of a bucket boundary, so the bar is the decode's, not equality)
        serving_step(0)
        out_two = out.clone()
        serving_step_one_call(0)
        torch.cuda.synchronize()
        extra["serving_one_call_max_abs_diff_from_two_calls"] = float((out.float() - out_two.float()).abs().max())
        del caches
        torch.cuda.empty_cache()
        rows_tok = 32 * 65536
        x = outlier_rows(rows_tok, H_KV, D, 1001, dev)
        packed = torch.empty(rows_tok, H_KV, D // 2, dtype=torch.uint8, device=dev)
        norms = torch.empty(rows_tok, H_KV, 1, device=dev)
        ev, od = C.split_rotation(rot)
        ev, od = ev.to(dev), od.to(dev)
        bnd_d = book[1]
        for _ in range(2):
            K.tq4_compress(x, rot_d, bnd_d, rotation_T_even=ev, rotation_T_odd=od, out=(packed, norms))
        c_ms, _ = time_events(lambda i: K.tq4_compress(x, rot_d, bnd_d, rotation_T_even=ev, rotation_T_odd=od,
                                                       out=(packed, norms)), EXTRA_ITERS)
        nrows = rows_tok * H_KV
        if check is not None:
            # the indices and norms of a sample of the rows just compressed, against the oracle
            ns = 2048
            idx_want, norms_want, _ = O.compress_indices(x[:ns].cpu(), rot, book[1].cpu())
            idx_got = O.nibble_unpack(packed[:ns].cpu())
            rate = (idx_got != idx_want).float().mean().item()
            nrel = ((norms[:ns].cpu() - norms_want).abs() / norms_want.clamp_min(1e-30)).max().item()
            check.update({"compress_index_mismatch_rate": rate, "compress_rows_checked": ns * H_KV,
                          "compress_norm_max_rel_err": nrel,
                          "compress_tolerance": "index mismatches on at most 1e-4 of the entries"})
            check["ok"] = bool(check["ok"] and rate <= 1e-4 and nrel <= 1e-5)
        extra.update({
            "compress_rows": nrows,
            "compress_ms": c_ms,
            "compress_mrows_per_s": nrows / (c_ms * 1e-3) / 1e6,
            "compress_mtok_per_s": rows_tok / (c_ms * 1e-3) / 1e6,
            "compress_gbps": nrows * 324 / (c_ms * 1e-3) / 1e9,
            "compress_pct_hbm_peak": 100.0 * nrows * 324 / (c_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            # bf16 rows against the 2-term bf16 split of the rotation: 2 x 2 D^2 flops per row on the MFMA
            "compress_matrix_terms": 2,
            "compress_tflops_bf16_mfma": nrows * 2 * 2 * D * D / (c_ms * 1e-3) / 1e12,
        })
        del x
        torch.cuda.empty_cache()
        y = torch.empty(rows_tok, H_KV, D, dtype=torch.bfloat16, device=dev)
        for _ in range(2):
            K.tq4_decompress(packed, norms, cent_d, torch.bfloat16, out=y)
        d_ms, _ = time_events(lambda i: K.tq4_decompress(packed, norms, cent_d, torch.bfloat16, out=y), EXTRA_ITERS)
        extra.update({
            "decompress_ms": d_ms,
            "decompress_gbps": nrows * 324 / (d_ms * 1e-3) / 1e9,
            "decompress_pct_hbm_peak": 100.0 * nrows * 324 / (d_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        })

        dr_ms, _ = time_events(lambda i: K.tq4_decompress_rotated(packed, norms, cent_d, rot_d, torch.bfloat16, out=y),
                               EXTRA_ITERS)
        extra.update({
            "decompress_rotated_ms": dr_ms,
            "decompress_rotated_gbps": nrows * 324 / (dr_ms * 1e-3) / 1e9,
            "decompress_rotated_pct_hbm_peak": 100.0 * nrows * 324 / (dr_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        })

        del y, packed, norms
        torch.cuda.empty_cache()

        # ---- fused TQ4 prefill (configs[3]): batch 4, 32 query heads over 8, 8192 tokens, causal ----
        pb, pn = 4, 8192
        gq3 = torch.Generator(device=dev).manual_seed(1003)
        q3 = torch.randn(pb, H_Q, pn, D, generator=gq3, device=dev).to(torch.bfloat16)
        kx = outlier_rows(pb * pn, H_KV, D, 1013, dev)            # (tokens, heads, D)
        vx = outlier_rows(pb * pn, H_KV, D, 1023, dev)
        kp3, kn3 = K.tq4_compress(kx, rot_d, bnd_d)
        vp3, vn3 = K.tq4_compress(vx, rot_d, bnd_d)
        # the same tokens in a paged cache behind a shuffled block table, for the paged prefill
        pages3 = pb * pn // BS
        cache3 = torch.zeros(pages3, BS, ROW_BYTES, dtype=torch.uint8, device=dev)
        table3 = torch.randperm(pages3, generator=torch.Generator().manual_seed(1033)).to(torch.int32)
        table3 = table3.reshape(pb, pn // BS).to(dev)
        t3 = torch.arange(pn, device=dev)
        slots3 = torch.cat([table3[b_i].long()[t3 // BS] * BS + t3 % BS for b_i in range(pb)])
        K.tq4_compress_and_store(kx, vx, rot_d, bnd_d, cache3, slots3)
        del kx, vx, slots3, t3

        def to_bhnd(t):                                            # (B*N, H, X) -> (B, H, N, X)
            return t.reshape(pb, pn, H_KV, -1).permute(0, 2, 1, 3).contiguous()

        kp3, kn3, vp3, vn3 = (to_bhnd(t) for t in (kp3, kn3, vp3, vn3))
        for _ in range(2):
            K.fused_tq_attention(q3, kp3, kn3, vp3, vn3, cent_d, cent_d, rot_d, sm_scale=scale, is_causal=True)
        p_ms, _ = time_events(lambda i: K.fused_tq_attention(q3, kp3, kn3, vp3, vn3, cent_d, cent_d, rot_d,
                                                             sm_scale=scale, is_causal=True), EXTRA_ITERS)
        p_flops = 4.0 * pn * pn * D * pb * H_Q / 2.0               # causal half of QK^T and PV
        extra.update({
            "prefill_ms": p_ms,
            "prefill_tflops": p_flops / (p_ms * 1e-3) / 1e12,
            "prefill_pct_fp16_mfma_peak": 100.0 * p_flops / (p_ms * 1e-3) / 2.5e15,
            "prefill_tokens_per_s": pb * pn / (p_ms * 1e-3),
        })
        q3v = q3.permute(0, 2, 1, 3).reshape(pb * pn, H_Q, D).contiguous()      # (tokens, heads, D)
        cu3 = torch.arange(pb + 1, dtype=torch.int32, device=dev) * pn
        lens3 = torch.full((pb,), pn, dtype=torch.int32, device=dev)
        out3 = torch.empty_like(q3v)

        def paged_prefill_step(i):
            K.paged_tq4_prefill(q3v, cu3, pn, cache3, table3, lens3, cent_d, cent_d, rot_d, H_KV, D, BS,
                                sm_scale=scale, causal=True, out=out3)

        for i in range(2):
            paged_prefill_step(i)
        pp_ms, _ = time_events(paged_prefill_step, EXTRA_ITERS)
        extra.update({
            "paged_prefill_ms": pp_ms,
            "paged_prefill_tflops": p_flops / (pp_ms * 1e-3) / 1e12,
            "paged_prefill_pct_fp16_mfma_peak": 100.0 * p_flops / (pp_ms * 1e-3) / 2.5e15,
        })
        del q3, q3v, out3, cache3, kp3, kn3, vp3, vn3
        torch.cuda.empty_cache()

        # ---- long-context decode over TurboQuantProd key / TQ4 value pages (configs[4]) ----------
        # batch 8, 64 query heads over 8, ragged contexts U{16K..128K} (seed 1004), 16-token pages
        hq4, b4 = 64, 8
        c3, b3 = C.codebook.solve_lloyd_max(D, 3)
        sk = C.qjl_matrix(D, 42)
        c3_d, b3_d, sk_d = c3.to(dev), b3.to(dev), sk.to(dev)
        g4 = torch.Generator(device="cpu").manual_seed(1004)
        lens4 = torch.randint(16384, 131072 + 1, (b4,), generator=g4)
        pages4 = (lens4 + BS - 1) // BS
        max_pages = int(pages4.max())
        total_pages = int(pages4.sum())
        row4 = K.prod_page_layout(H_KV, D)[4]
        cache4 = torch.zeros(total_pages, BS, row4, dtype=torch.uint8, device=dev)
        perm = torch.randperm(total_pages, generator=g4)
        table4 = torch.zeros(b4, max_pages, dtype=torch.int32)
        w_rot = None
        first = 0
        for s_i in range(b4):
            L = int(lens4[s_i])
            npg = int(pages4[s_i])
            table4[s_i, :npg] = perm[first:first + npg].to(torch.int32)
            first += npg
            t = torch.arange(L)
            slots = (table4[s_i].long()[t // BS] * BS + t % BS).to(dev)
            kx = outlier_rows(L, H_KV, D, 1400 + s_i, dev)
            vx = outlier_rows(L, H_KV, D, 1500 + s_i, dev)
            kp4, kn4, kg4 = K.prod_compress(kx, rot_d, sk_d, b3_d, c3_d)
            vp4, vn4 = K.tq4_compress(vx, rot_d, bnd_d)
            K.prod_store_rows(cache4, slots, kp4, kn4, kg4, vp4, vn4)
            del kx, vx, kp4, kn4, kg4, vp4, vn4
        table4 = table4.to(dev)
        lens4_d = lens4.to(torch.int32).to(dev)
        q4 = torch.randn(b4, hq4, D, generator=torch.Generator(device="cpu").manual_seed(1044)).to(torch.bfloat16).to(dev)
        out4 = torch.empty_like(q4)

        def prod_step(i):
            K.prod_paged_decode(q4, cache4, table4, lens4_d, c3_d, cent_d, rot_d, sk_d, H_KV, D, BS,
                                sm_scale=scale, out=out4)

        for i in range(3):
            prod_step(i)
        pd_ms, _ = time_events(prod_step, EXTRA_ITERS)
        prod_bytes = int(lens4.sum()) * row4
        extra.update({
            "prod_decode_ms": pd_ms,
            "prod_decode_gbps": prod_bytes / (pd_ms * 1e-3) / 1e9,
            "prod_decode_pct_hbm_peak": 100.0 * prod_bytes / (pd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "prod_decode_tokens_per_s": b4 / (pd_ms * 1e-3),
            "prod_context_tokens": int(lens4.sum()),
            "prod_bytes_per_token_per_kv_head": row4 // H_KV,
            "prod_cache_bytes": prod_bytes,
        })
        del cache4, q4, out4, table4
        torch.cuda.empty_cache()

        # ---- the same operators on other shapes (not BASELINE configs; shapes the reference's launchers
        # also take: csrc/cuda/paged_decode.cu:401-415, fused_tq_attention.cu:497-506) -----------------
        def decode_shape(n_seq, ctx, hq, hkv, d, n_caches=2):
            cent_s, bnd_s = C.codebook.solve_lloyd_max(d, 4)
            rot_s = C.haar_orthogonal(d, 42).to(dev)
            cent_s, bnd_s = cent_s.to(dev), bnd_s.to(dev)
            row = hkv * (d + 8)
            pages = n_seq * ctx // BS
            made = []
            for i in range(n_caches):
                kx = torch.randn(n_seq * ctx, hkv, d, device=dev).to(torch.bfloat16)
                vx = torch.randn(n_seq * ctx, hkv, d, device=dev).to(torch.bfloat16)
                cache_s = torch.zeros(pages, BS, row, dtype=torch.uint8, device=dev)
                tab = torch.randperm(pages, generator=torch.Generator().manual_seed(70 + i)).reshape(n_seq, ctx // BS)
                tab = tab.to(torch.int32).to(dev)
                t = torch.arange(ctx, device=dev)
                slots = (tab.long()[:, t // BS] * BS + (t % BS)).reshape(-1)
                K.tq4_compress_and_store(kx, vx, rot_s, bnd_s, cache_s, slots)
                made.append((cache_s, tab))
                del kx, vx
            qs = torch.randn(n_seq, hq, d, device=dev).to(torch.bfloat16)
            ls = torch.full((n_seq,), ctx, dtype=torch.int32, device=dev)
            os_ = torch.empty_like(qs)

            def f(i):
                c_, t_ = made[i % n_caches]
                K.split_k_paged_decode(qs, c_, t_, ls, cent_s, cent_s, rot_s, hkv, d, BS, sm_scale=1.0 / math.sqrt(d), out=os_)

            for i in range(30):
                f(i)
            ms, _ = time_events(f, 40)
            return ms, n_seq * ctx * row

        def prefill_shape(b, n, hq, hkv, d):
            cent_s, bnd_s = C.codebook.solve_lloyd_max(d, 4)
            rot_s = C.haar_orthogonal(d, 42).to(dev)
            cent_s, bnd_s = cent_s.to(dev), bnd_s.to(dev)
            qx = torch.randn(b, hq, n, d, device=dev).to(torch.bfloat16)
            kx = torch.randn(b * n, hkv, d, device=dev).to(torch.bfloat16)
            vx = torch.randn(b * n, hkv, d, device=dev).to(torch.bfloat16)
            kp_, kn_ = K.tq4_compress(kx, rot_s, bnd_s)
            vp_, vn_ = K.tq4_compress(vx, rot_s, bnd_s)

            def bhnd(t_):
                return t_.reshape(b, n, hkv, -1).permute(0, 2, 1, 3).contiguous()

            kp_, kn_, vp_, vn_ = (bhnd(t_) for t_ in (kp_, kn_, vp_, vn_))

            def f(i):
                K.fused_tq_attention(qx, kp_, kn_, vp_, vn_, cent_s, cent_s, rot_s, sm_scale=1.0 / math.sqrt(d), is_causal=True)

            for i in range(2):
                f(i)
            ms, _ = time_events(f, 5)
            return ms, 4.0 * n * n * d * b * hq / 2

        shapes = {}
        for name, (n_seq, ctx, hq, hkv, d) in ({} if args.skip_other_shapes else {
            "decode_32x16384_32q_8kv_d128": (32, 16384, 32, 8, 128),
            "decode_32x4096_32q_4kv_d128": (32, 4096, 32, 4, 128),
            "decode_128x8192_8q_1kv_d128": (128, 8192, 8, 1, 128),      # a tensor-parallel shard of a model with 8 KV heads
            "decode_32x4096_8q_1kv_d128": (32, 4096, 8, 1, 128),
            "decode_128x8192_16q_2kv_d128": (128, 8192, 16, 2, 128),
            "decode_32x4096_32q_8kv_d64": (32, 4096, 32, 8, 64),
            "decode_32x4096_32q_8kv_d256": (32, 4096, 32, 8, 256),
            "decode_32x4096_8q_1kv_d256": (32, 4096, 8, 1, 256),        # one KV head of 256 coordinates
            "decode_32x4096_16q_4kv_d64": (32, 4096, 16, 4, 64),
        }).items():
            ms, nbytes = decode_shape(n_seq, ctx, hq, hkv, d)
            shapes[name] = {"step_us": ms * 1e3, "gbps": nbytes / (ms * 1e-3) / 1e9,
                            "pct_hbm_peak": 100.0 * nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
            torch.cuda.empty_cache()
        for name, (b, n, hq, hkv, d) in ({} if args.skip_other_shapes else {
            "prefill_2x8192_32q_8kv_d64": (2, 8192, 32, 8, 64),
            "prefill_2x8192_16q_4kv_d256": (2, 8192, 16, 4, 256),
        }).items():
            ms, flops = prefill_shape(b, n, hq, hkv, d)
            shapes[name] = {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12,
                            "pct_fp16_mfma_peak": 100.0 * flops / (ms * 1e-3) / 2.5e15}
            torch.cuda.empty_cache()
        if shapes:
            extra["other_shapes"] = shapes

    value = kv_bytes / (step_ms * 1e-3) / 1e9
    traffic, traffic_src = committed_traffic(DOMINANT_KERNEL)
    line = {
        "metric": "tq4_paged_decode_hbm_gbps",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "configs[2]: split-K paged TQ4 decode, Llama-3-8B layer shape",
            "batch": BATCH, "context": CTX, "q_heads": H_Q, "kv_heads": H_KV, "head_dim": D,
            "page_tokens": BS, "query_dtype": "bf16", "cache": "cold (4 caches of 143 MB in rotation)",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            # HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by a plain copy, as the
            # committed counter summary states them for this kernel (null when it does not cover it)
            "traffic": traffic,
            "traffic_source": traffic_src,
            "kernel": DOMINANT_KERNEL,
        },
        "cpu_baseline": cpu,
        "check": check,
        "check_ok": None if check is None else check["ok"],
        "check_max_abs_err": None if check is None else check["max_abs_err"],
        "decode_step_us_wallclock": wall_ms * 1e3,
        "extra": extra,
    }
    print(json.dumps(line), flush=True)
    if check is not None and not check["ok"]:
        log("bench.py: the output check against the oracle FAILED:", json.dumps(check))
        sys.exit(1)


if __name__ == "__main__":
    main()
