#!/usr/bin/env python3
"""Headline benchmark: paged TQ4 decode attention at 128K context on one MI355X.

One "step" = one full-attention layer's decode attention for the workload
(`warp34_paged_attention_bf16` over TQ4 pages, through the C ABI).  The KV pools of
several layers are allocated and the steps cycle through them, as a decode step of the model
would, so that the working set (layers x 69.2 MB) exceeds the 256 MB last-level cache and
the figure is an HBM figure.  K/V are synthetic bf16 N(0,1) with 1 % outlier channels (x20),
TQ4-encoded by the library's own quantize-on-append kernel into 64-token pages whose
physical order is a seeded permutation.  Every input comes from the library's deterministic
generators (include/warp34_synth.h: SplitMix64 -> Box-Muller -> bf16, Fisher-Yates), so two
machines build the same bytes.

Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
KV_HEADS, Q_HEADS, HEAD_DIM, BLOCK = 2, 16, 256, 64
ROW_BYTES = {"tq4": 132, "bf16": 512, "fp8": 264, "q8_0": 272}
WORKLOADS = {
    # name: (kv format, context lengths or None for the seeded 32-sequence draw, pool tokens)
    "tq4_decode_b1_ctx131072": ("tq4", [131072], 0),
    "tq4_decode_b8_ctx131072": ("tq4", [131072] * 8, 0),
    "tq4_decode_b32_ctx1k_64k": ("tq4", None, 2 << 20),
    "bf16_decode_b1_ctx32768": ("bf16", [32768], 0),
    "bf16_decode_b16_ctx32768": ("bf16", [32768] * 16, 0),
    # the un-rotated 8-bit rows the default TQ4 policy keeps for its last four layers
    "fp8_decode_b1_ctx131072": ("fp8", [131072], 0),
    "q8_0_decode_b1_ctx131072": ("q8_0", [131072], 0),
    "fp8_decode_b32_ctx1k_64k": ("fp8", None, 2 << 20),
    # 8 sequences, 16 384-token TQ4 prefix + 2 048-token bf16 chunk each: append + causal attention
    "tq4_prefill_8x2048_ctx16384": ("tq4", [18432] * 8, 0),
    "fp8_prefill_8x2048_ctx16384": ("fp8", [18432] * 8, 0),
    "bf16_prefill_8x2048_ctx16384": ("bf16", [18432] * 8, 0),
    "q8_0_prefill_8x2048_ctx16384": ("q8_0", [18432] * 8, 0),
    # quantize-on-append alone: 4 096 tokens x 2 kv heads (K and V) from bf16 into 64-token TQ4 pages
    "tq4_append_4096": ("tq4", [4096], 0),
    # producer side: QK RMSNorm + RoPE fused with the TQ4 append of an 8 192-token chunk
    "tq4_norm_rope_append_8192": ("tq4", [8192], 0),
    # the target model's producer: Gemma RMSNorm + interleaved mRoPE + gate split fused with the TQ4 append
    "tq4_fused_qk_gate_append_8192": ("tq4", [8192], 0),
    # consumer side: out = attn_out * sigmoid(gate) over the rows of a 16 384-token prefill step
    "attn_output_gate_16384x4096": ("tq4", [64], 0),
    # QSA sparse attention: 1, 16 or 256 query tokens, each over its own 513 selected 4-token groups (2 052 keys)
    # of a 131 072-token sequence
    "tq4_qsa_sparse_1x513_ctx131072": ("tq4", [131072], 0),
    "tq4_qsa_sparse_16x513_ctx131072": ("tq4", [131072], 0),
    "tq4_qsa_sparse_256x513_ctx131072": ("tq4", [131072], 0),
    "fp8_qsa_sparse_16x513_ctx131072": ("fp8", [131072], 0),
    # 16 sequences of 262 144 tokens that share the pages of a 200 000-token prefix; 4 query tokens each
    "tq4_verify_16x4_ctx262144_shared200k": ("tq4", [262144] * 16, 0),
}
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs scaled by
# a plain copy of known size (the scale is stated in each profile); counters cannot
# be read from inside this process, so workloads without such a profile report null.
PROFILED_TRAFFIC = {
    # workload: (HBM bytes per launch of the dominant kernel, the profile that holds the counter readings)
    "tq4_decode_b1_ctx131072": (71_820_000, "profiles/paged_attn_tq4_decode_b1_ctx131072.txt"),
    "tq4_decode_b8_ctx131072": (559_960_000, "profiles/paged_attn_tq4_decode_b8_ctx131072.txt"),
    "tq4_decode_b32_ctx1k_64k": (587_160_000, "profiles/paged_attn_tq4_decode_b32_ctx1k_64k.txt"),
    "bf16_decode_b1_ctx32768": (69_520_000, "profiles/paged_attn_rows_bf16_decode_b1_ctx32768.txt"),
    "fp8_decode_b32_ctx1k_64k": (1_190_120_000, "profiles/paged_attn_rows_fp8_decode_b32_ctx1k_64k.txt"),
    "fp8_decode_b1_ctx131072": (142_290_000, "profiles/paged_attn_rows_fp8_decode_b1_ctx131072.txt"),
    "q8_0_decode_b1_ctx131072": (145_300_000, "profiles/paged_attn_rows_q8_0_decode_b1_ctx131072.txt"),
    # (the four kernels of the shared-prefix path together: probe 0.27 + tile 144.84 + decode 534.98 + merge 39.06 MB)
    "tq4_verify_16x4_ctx262144_shared200k": (719_150_000, "profiles/paged_attn_tq4_verify_16x4_ctx262144_shared200k.txt"),
    "tq4_prefill_8x2048_ctx16384": (1_119_610_000, "profiles/paged_prefill_tq4_8x2048_ctx16384.txt"),
    "tq4_qsa_sparse_16x513_ctx131072": (23_400_000, "profiles/qsa_sparse_tq4_16x513_ctx131072.txt"),
    "tq4_norm_rope_append_8192": (182_920_000, "profiles/qk_norm_rope_tq4_append_8192.txt"),
    "tq4_fused_qk_gate_append_8192": (289_660_000, "profiles/fused_qk_norm_rope_gate_tq4_append_8192.txt"),
    "tq4_append_4096": (10_880_000, "profiles/kv_append_tq4_4096.txt"),
}
SHARED_PREFIX = {"tq4_verify_16x4_ctx262144_shared200k": 200000}
VERIFY_Q = {"tq4_verify_16x4_ctx262144_shared200k": 4}
PREFILL_CHUNK = 2048


def dev_bf16(torch, bits):
    """uint16 bf16 bits (numpy) -> bf16 tensor on the device"""
    return torch.from_numpy(bits.view(np.int16)).to("cuda:0").view(torch.bfloat16)


def synth_normal(torch, ffi, shape, seed, dtype=None):
    """N(0,1) tensor on the device from the library's generator (bf16 values, optionally cast)."""
    n = int(np.prod(shape))
    t = dev_bf16(torch, ffi.synth_normal_bf16(n + (n & 1), seed)[:n]).reshape(shape)
    return t if dtype is None else t.to(dtype)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed steps (default 200; 10 for the prefill workload)")
    ap.add_argument("--warmup", type=int, default=-1, help="untimed steps (default 20; 2 for the prefill workload)")
    ap.add_argument("--condition-ms", type=float, default=150.0, dest="condition_ms",
                    help="run the workload untimed for this long before the warm-up steps, so that the GPU "
                         "clocks are at their sustained state (0 = off)")
    ap.add_argument("--workload", default="tq4_decode_b1_ctx131072",
                    choices=sorted(WORKLOADS))
    ap.add_argument("--ctx", type=int, default=0, help="override: one request with this context length")
    ap.add_argument("--layers", type=int, default=0, help="KV pools to cycle through (0 = auto, > 256 MB total)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-batch-point", action="store_true",
                    help="headline workload only: skip the additional 8-sequence measurement")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run plain 256 MiB device copies instead of a workload (scale reference for the "
                         "FETCH_SIZE / WRITE_SIZE counters of rocprofv3 --pmc)")
    args = ap.parse_args()
    prefill = "_prefill_" in args.workload
    if args.steps <= 0:
        args.steps = 10 if prefill else 200
    if args.warmup < 0:
        args.warmup = 2 if prefill else 20
    return args


def build_workload(name, seed=0):
    fmt, ctx, pool_tokens = WORKLOADS[name]
    if ctx is None:  # 32 context lengths drawn uniformly from 1K .. 64K
        from warp34_amd import ffi

        ctx = ffi.synth_uniform_i32(32, 1024, 65536, seed)
    return fmt, np.asarray(ctx, dtype=np.int64), pool_tokens


class Layer:
    """One layer's KV pool on the device, filled through the append kernel."""

    def __init__(self, torch, lib, ffi, fmt, ctx, pool_pages, seed, shared_prefix=0):
        dev = "cuda:0"
        self.tok, self.head = ROW_BYTES[fmt], BLOCK * ROW_BYTES[fmt]
        self.page = KV_HEADS * self.head
        self.k = torch.zeros(pool_pages * self.page, dtype=torch.uint8, device=dev)
        self.v = torch.zeros(pool_pages * self.page, dtype=torch.uint8, device=dev)
        kv_format = {"tq4": ffi.WARP34_KV_FORMAT_TQ4, "bf16": ffi.WARP34_KV_FORMAT_BF16,
                     "fp8": ffi.WARP34_KV_FORMAT_FP8_E4M3, "q8_0": ffi.WARP34_KV_FORMAT_Q8_0}[fmt]
        xf = ffi.WARP34_KV_TRANSFORM_RADEMACHER_WHT256 if fmt == "tq4" else ffi.WARP34_KV_TRANSFORM_IDENTITY
        self.layout = ffi.Warp34KvLayerLayout(
            self.k.data_ptr(), self.v.data_ptr(), self.page, self.head, self.tok, self.page, self.head, self.tok,
            0, seed, KV_HEADS, HEAD_DIM, BLOCK, kv_format, kv_format, xf, xf, 0)
        pages_per = [(int(c) + BLOCK - 1) // BLOCK for c in ctx]
        perm = torch.from_numpy(ffi.synth_permutation(pool_pages, 1000 + seed)).to(dev)
        mb = max(pages_per)
        bt = torch.zeros((len(ctx), mb), dtype=torch.int32, device=dev)
        at = 0
        shared_pages = shared_prefix // BLOCK  # whole pages, owned by request 0
        for r, n in enumerate(pages_per):
            if r > 0 and shared_pages:
                bt[r, :shared_pages] = bt[0, :shared_pages]
                bt[r, shared_pages:n] = perm[at:at + n - shared_pages]
                at += n - shared_pages
            else:
                bt[r, :n] = perm[at:at + n]
                at += n
        self.block_tables = bt
        self.max_blocks = mb
        # K and V rows: one stream per layer and tensor (3 of 256 channels per kv head x20), the
        # requests' tokens one after the other
        k_seed, v_seed = 10 * seed + 1, 10 * seed + 2
        stream = torch.cuda.current_stream().cuda_stream
        ex = ffi.Warp34Exec(stream, 0, 0, 0)
        chunk = 2048
        self.tail_k, self.tail_v, self.tail_slots = [], [], []
        row_at = 0
        for r, c in enumerate(ctx):
            c = int(c)
            first = shared_pages * BLOCK if r > 0 else 0  # shared pages were filled by request 0
            k_all = dev_bf16(torch, ffi.synth_kv_rows_bf16(c - first, KV_HEADS, HEAD_DIM, k_seed, 3, first_row=row_at))
            v_all = dev_bf16(torch, ffi.synth_kv_rows_bf16(c - first, KV_HEADS, HEAD_DIM, v_seed, 3, first_row=row_at))
            row_at += c - first
            for t0 in range(first, c, chunk):
                n = min(chunk, c - t0)
                kk = k_all[t0 - first:t0 - first + n]
                vv = v_all[t0 - first:t0 - first + n]
                pos = torch.arange(t0, t0 + n, device=dev)
                slots = (bt[r, (pos // BLOCK)].to(torch.int64) * BLOCK + pos % BLOCK).to(torch.int32)
                qsl = torch.tensor([0, n], dtype=torch.int32, device=dev)
                seq = torch.tensor([t0 + n], dtype=torch.int32, device=dev)
                b = ffi.Warp34AttentionBatch(qsl.data_ptr(), None, seq.data_ptr(), bt[r].data_ptr(), slots.data_ptr(),
                                             None, None, 1, n, mb, n, t0 + n, 0, 0, 0.0625, 0)
                rc = lib.warp34_kv_cache_write_bf16(C.byref(ex), C.byref(self.layout), C.byref(b),
                                                    C.c_void_p(kk.data_ptr()), C.c_void_p(vv.data_ptr()))
                if rc:
                    raise RuntimeError("warp34_kv_cache_write_bf16 rc=%d" % rc)
                torch.cuda.synchronize()
                if t0 + n == c:  # the request's last chunk, re-appended by the prefill workload
                    self.tail_k.append(kk)
                    self.tail_v.append(vv)
                    self.tail_slots.append(slots)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(torch, sample, threads, min_seconds=1.5):
    """The CPU oracle (restatement of the reference's scalar path) timed on this host over the SAME
    workload the GPU leg ran: layer 0's pages as the append kernel wrote them (downloaded),
    its block table, the same queries; all host threads up to 16.  Also reports how far the GPU
    output is from the oracle's.  Requests beyond a bound on the total context are left out of
    the sample (said in `sample`)."""
    import oracle

    L, q, ctx, ql, fmt, got = sample["layer"], sample["q"], sample["ctx"], sample["ql"], sample["fmt"], sample["out"]
    ofmt = {"tq4": oracle.FMT_TQ4, "bf16": oracle.FMT_BF16, "fp8": oracle.FMT_FP8, "q8_0": oracle.FMT_Q8_0}[fmt]
    xf = oracle.XF_WHT256 if fmt == "tq4" else oracle.XF_IDENTITY
    # bounded sample: leading requests up to 262 144 context tokens in total
    keep, tot = 0, 0
    for c in ctx:
        if keep and tot + int(c) > 262144:
            break
        keep, tot = keep + 1, tot + int(c)
    pool_pages = L.k.numel() // L.page
    pool = oracle.HostPool(pool_pages, KV_HEADS, HEAD_DIM, BLOCK, ofmt, xf)
    pool.k[:] = L.k.cpu().numpy()
    pool.v[:] = L.v.cpu().numpy()
    bt = L.block_tables[:keep].cpu().numpy()
    qsl = [ql * r for r in range(keep + 1)]
    seq = [int(c) for c in ctx[:keep]]
    hb = oracle.HostBatch(qsl, seq, bt, context_lens_before=[c - ql for c in seq])
    qb = q[:keep * ql].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    # append rate: 4 096 rows, single thread
    rows = 4096
    kk = oracle.fill_kv_rows(rows // (2 * KV_HEADS), KV_HEADS, HEAD_DIM, 1, oracle.DT_BF16, 3)
    small = oracle.HostPool(rows // (2 * KV_HEADS) // BLOCK, KV_HEADS, HEAD_DIM, BLOCK, ofmt, xf)
    bt_s = np.arange(small.k.size // (KV_HEADS * BLOCK * ROW_BYTES[fmt]), dtype=np.int32).reshape(1, -1)
    n_s = rows // (2 * KV_HEADS)
    wb = oracle.HostBatch([0, n_s], [n_s], bt_s, context_lens_before=[0],
                          write_slot_mapping=oracle.slot_mapping(bt_s[0], 0, n_s, BLOCK))
    t0 = time.perf_counter()
    oracle.kv_cache_write(small, wb, kk, kk, oracle.DT_BF16)
    t_append = time.perf_counter() - t0
    # the same append on all threads: every thread appends its own 4 096 rows into its own pages
    # (the oracle's append is a plain C loop over rows; ctypes releases the interpreter lock)
    from concurrent.futures import ThreadPoolExecutor

    pools = [oracle.HostPool(rows // (2 * KV_HEADS) // BLOCK, KV_HEADS, HEAD_DIM, BLOCK, ofmt, xf) for _ in range(threads)]
    with ThreadPoolExecutor(threads) as ex:
        list(ex.map(lambda pl: oracle.kv_cache_write(pl, wb, kk, kk, oracle.DT_BF16), pools))  # warm-up
        t0 = time.perf_counter()
        list(ex.map(lambda pl: oracle.kv_cache_write(pl, wb, kk, kk, oracle.DT_BF16), pools))
        t_append_all = time.perf_counter() - t0
    # decode on one thread: one run (16 x the time of the all-threads run)
    t0 = time.perf_counter()
    oracle.paged_attention(pool, hb, qb, oracle.DT_BF16, Q_HEADS, n_threads=1)
    t_one = time.perf_counter() - t0
    reps, t_total, want = 0, 0.0, None
    while t_total < min_seconds:
        t0 = time.perf_counter()
        want = oracle.paged_attention(pool, hb, qb, oracle.DT_BF16, Q_HEADS, n_threads=threads)
        t_total += time.perf_counter() - t0
        reps += 1
    dt = t_total / reps
    kv_bytes = tot * KV_HEADS * 2 * ROW_BYTES[fmt]
    gotf = got[:keep * ql].float().cpu().numpy().astype(np.float64)
    err = np.abs(gotf - np.asarray(want, dtype=np.float64))
    return {
        "value": round(kv_bytes / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "CPU oracle (oracle/tq4_oracle.c) over the same workload: layer 0's pages as written by the append "
                  "kernel, %d of %d requests (%d context tokens), %d query token(s) each, %d pthreads on %s "
                  "(%d hardware threads): %.1f ms/layer, mean of %d runs; the same on 1 thread: %.1f ms/layer; append of "
                  "%d rows: %.0f rows/s on 1 thread, %.0f rows/s on %d threads"
                  % (keep, len(ctx), tot, ql, threads, cpu_model(), os.cpu_count() or 0, dt * 1e3, reps, t_one * 1e3, rows,
                     rows / t_append, threads * rows / t_append_all, threads),
        "us_per_layer": round(dt * 1e6, 1),
        # the four legs: decode and append, one thread and all threads (`value` is decode on all threads)
        "legs": {
            "decode_all_threads": {"threads": threads, "GBps": round(kv_bytes / dt / 1e9, 4), "us_per_layer": round(dt * 1e6, 1)},
            "decode_1_thread": {"threads": 1, "GBps": round(kv_bytes / t_one / 1e9, 4), "us_per_layer": round(t_one * 1e6, 1)},
            "append_1_thread": {"threads": 1, "rows_per_s": round(rows / t_append), "rows": rows},
            "append_all_threads": {"threads": threads, "rows_per_s": round(threads * rows / t_append_all),
                                   "rows": threads * rows},
        },
        "gpu_vs_oracle": {"max_abs_err": float(err.max()), "max_rel": float(err.max() / max(np.abs(want).max(), 1e-30)),
                          "worst_excess_over_2e-3_plus_1e-2_want": float((err - (2e-3 + 1e-2 * np.abs(want))).max())},
    }


def run_prefill(args, torch, lib, ffi, layers, ctx, n_layers, pool_pages, fmt):
    """Chunked prefill: every sequence re-appends its last PREFILL_CHUNK tokens (bf16 -> TQ4 / FP8)
    and attends causally over prefix + chunk.  One step = append + attention of one layer."""
    dev = "cuda:0"
    R, n = len(ctx), PREFILL_CHUNK
    N = R * n
    q = synth_normal(torch, ffi, (N, Q_HEADS, HEAD_DIM), 7)
    out = torch.zeros_like(q)
    qsl = (torch.arange(0, R + 1, dtype=torch.int32, device=dev) * n).to(torch.int32)
    seq = torch.tensor(ctx, dtype=torch.int32, device=dev)
    ctxb = (seq - n).to(torch.int32)
    scratch_bytes = 32 << 20
    scratch = torch.zeros(scratch_bytes, dtype=torch.uint8, device=dev)
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, scratch.data_ptr(), scratch_bytes, 0)
    per_layer = []
    for L in layers:
        kk, vv, slots = torch.cat(L.tail_k), torch.cat(L.tail_v), torch.cat(L.tail_slots)
        batch = ffi.Warp34AttentionBatch(
            qsl.data_ptr(), ctxb.data_ptr(), seq.data_ptr(), L.block_tables.data_ptr(), slots.data_ptr(), None, None,
            R, N, L.max_blocks, n, int(ctx.max()), 0, 0, 1.0 / 16.0, 0)
        per_layer.append((L, kk, vv, slots, batch))

    def step(i, append=True):
        L, kk, vv, slots, batch = per_layer[i % n_layers]
        if append:
            rc = lib.warp34_kv_cache_write_bf16(C.byref(ex), C.byref(L.layout), C.byref(batch),
                                                C.c_void_p(kk.data_ptr()), C.c_void_p(vv.data_ptr()))
            if rc:
                raise RuntimeError("warp34_kv_cache_write_bf16 rc=%d" % rc)
        rc = lib.warp34_paged_attention_bf16(C.byref(ex), C.byref(L.layout), C.byref(batch),
                                             C.c_void_p(q.data_ptr()), C.c_void_p(out.data_ptr()), Q_HEADS)
        if rc:
            raise RuntimeError("warp34_paged_attention_bf16 rc=%d" % rc)

    def timed(append):
        condition(args, torch, lambda i: step(i, append))
        for i in range(args.warmup):
            step(i, append)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.steps):
            step(i, append)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms_attn = timed(False)
    ms_step = timed(True)
    assert torch.isfinite(out.float()).all()
    # QK^T and PV: 2 x 2 x head_dim flops per (query row, visible key)
    pairs = sum(sum(int(c) - n + i + 1 for i in range(n)) for c in ctx)
    flops = 4.0 * HEAD_DIM * Q_HEADS * pairs
    tf_step = flops / (ms_step * 1e-3) / 1e12
    tf_attn = flops / (ms_attn * 1e-3) / 1e12
    peak = 2500.0
    print(json.dumps({
        "metric": "chunked prefill over %s pages (append + causal attention): ms/layer + achieved MFMA TFLOP/s"
                  % fmt.upper(),
        "value": round(tf_step, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "ms_attention_only": round(ms_attn, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 MFMA operands (%s), f32 accumulate, bf16 Q/out"
                 % {"tq4": "TQ4 codes -> fp16 centroids", "fp8": "E4M3 codes widened",
                    "q8_0": "fp16(d * int8 code)"}.get(fmt, "rows as stored"),
        "data": "synthetic",
        "config": {"workload": args.workload, "requests": R, "chunk_tokens": n, "prefix_tokens": int(ctx[0]) - n,
                   "q_heads": Q_HEADS, "kv_heads": KV_HEADS, "head_dim": HEAD_DIM, "page_tokens": BLOCK,
                   "kv_format": "tq4+wht256" if fmt == "tq4" else fmt, "kv_pools_cycled": n_layers,
                   "pool_pages": pool_pages,
                   "attention_flops_per_step": flops, "rows_appended_per_step": N * KV_HEADS * 2},
        "roofline": {"bound": "mfma", "achieved": round(tf_attn, 1), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(tf_attn / peak, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
                     "kernel": "paged_prefill_tq4_kernel (attention-only launches)",
                     "avg_launch_us": round(ms_attn * 1e3, 1)},
    }))


def run_gate(args, torch, lib, ffi):
    """out = attn_out * sigmoid(gate) on fp16 [16 384, 4 096] (16 q heads x 256): three buffer sets
    are cycled so that the 403 MB of a step do not come out of the Infinity Cache."""
    dev = "cuda:0"
    n, dim, sets = 16384, Q_HEADS * HEAD_DIM, 3
    bufs = [tuple(synth_normal(torch, ffi, (n, dim), 50 + 2 * i + j, torch.float16) for j in range(2)) +
            (torch.empty((n, dim), dtype=torch.float16, device=dev),) for i in range(sets)]
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, 0, 0, 0)

    def step(i):
        a, gt, o = bufs[i % sets]
        rc = lib.warp34_apply_attn_output_gate_f16(C.byref(ex), C.c_void_p(a.data_ptr()), C.c_void_p(gt.data_ptr()),
                                                   C.c_void_p(o.data_ptr()), None, n, dim)
        if rc:
            raise RuntimeError("warp34_apply_attn_output_gate_f16 rc=%d" % rc)

    condition(args, torch, step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    nbytes = 3 * n * dim * 2
    gbs = nbytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "attention output gate: us/step + achieved HBM GB/s", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6),
        "us_per_layer": round(ms * 1e3, 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 arithmetic on f16 rows", "data": "synthetic",
        "config": {"workload": args.workload, "tokens": n, "total_dim": dim, "bytes_per_step": nbytes},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1], "kernel": "attn_output_gate_kernel<true>",
                     "avg_launch_us": round(ms * 1e3, 2)},
    }))


def run_qsa(args, torch, lib, ffi, layers, ctx_len, n_layers, n_tok, fmt, select_k=513):
    """QSA sparse paged attention (gate included): every query token attends over select_k 4-token groups
    drawn from the sequence's groups (the last group always among them, as the selector keeps the
    newest keys).  Algorithmic bytes = the selected K and V rows of both kv heads + the gate rows."""
    dev = "cuda:0"
    q = synth_normal(torch, ffi, (n_tok, Q_HEADS, HEAD_DIM), 23, torch.float16)
    gate = synth_normal(torch, ffi, (n_tok, Q_HEADS, HEAD_DIM), 24, torch.float16)
    out = torch.zeros_like(q)
    n_groups = ctx_len // 4
    gpp = BLOCK // 4
    per_layer = []
    for li, L in enumerate(layers):
        logs = torch.stack([torch.cat([
            torch.from_numpy(ffi.synth_permutation(n_groups - 1, 3000 + 1000 * li + t)[:select_k - 1].astype(np.int64)).to(dev),
            torch.tensor([n_groups - 1], device=dev)]) for t in range(n_tok)])
        phys = L.block_tables[0, (logs * 4 // BLOCK)].to(torch.int64) * gpp + (logs * 4 % BLOCK) // 4
        per_layer.append((phys.to(torch.int32).contiguous(), logs.to(torch.int32).contiguous()))
    num_sel = torch.full((n_tok,), select_k, dtype=torch.int32, device=dev)
    seq_pos = torch.full((n_tok,), ctx_len - 1, dtype=torch.int32, device=dev)
    scratch_bytes = 32 << 20
    scratch = torch.zeros(scratch_bytes, dtype=torch.uint8, device=dev)
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, scratch.data_ptr(), scratch_bytes, 0)
    vp = lambda t: C.c_void_p(t.data_ptr())

    def step(i):
        L = layers[i % n_layers]
        phys, logs = per_layer[i % n_layers]
        rc = lib.warp34_qsa_sparse_paged_attn_f16(C.byref(ex), vp(q), vp(gate), C.byref(L.layout), vp(phys), vp(logs),
                                                  vp(num_sel), vp(seq_pos), None, vp(out), n_tok, Q_HEADS, select_k,
                                                  1.0 / 16.0)
        if rc:
            raise RuntimeError("warp34_qsa_sparse_paged_attn_f16 rc=%d" % rc)

    condition(args, torch, step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    ms = e0.elapsed_time(e1) / args.steps
    keys = n_tok * select_k * 4
    nbytes = keys * KV_HEADS * 2 * ROW_BYTES[fmt] + n_tok * Q_HEADS * HEAD_DIM * 2
    gbs = nbytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "QSA sparse paged attention over %s pages: us/layer + achieved HBM GB/s" % fmt.upper(), "value": round(gbs, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6),
        "us_per_layer": round(ms * 1e3, 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 MFMA operands (%s), f32 accumulate, f16 Q/gate/out" %
                 ("TQ4 codes -> fp16 centroids" if fmt == "tq4" else "E4M3 codes widened, fp32 block scales"),
        "data": "synthetic",
        "config": {"workload": args.workload, "query_tokens": n_tok, "selected_groups_per_token": select_k,
                   "keys_per_token": select_k * 4, "context_tokens": ctx_len, "q_heads": Q_HEADS, "kv_heads": KV_HEADS,
                   "head_dim": HEAD_DIM, "page_tokens": BLOCK, "kv_format": "tq4+wht256" if fmt == "tq4" else fmt,
                   "kv_pools_cycled": n_layers, "bytes_per_step": nbytes},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
                     "kernel": ("qsa_sparse_tq4_kernel" if fmt == "tq4" else "qsa_sparse_rows_kernel") +
                               " + qsa_sparse_merge_kernel (whole call)",
                     "avg_launch_us": round(ms * 1e3, 2)},
    }))


def run_append(args, torch, lib, ffi, layers, n, n_layers, fmt):
    """Quantize-on-append alone: n tokens x KV_HEADS (K and V) of bf16 rows into the pages of one
    layer, the layers cycled.  One step = one layer's append of an n-token chunk."""
    dev = "cuda:0"
    k = synth_normal(torch, ffi, (n, KV_HEADS * HEAD_DIM), 21)
    v = synth_normal(torch, ffi, (n, KV_HEADS * HEAD_DIM), 22)
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, 0, 0, 0)
    per_layer = []
    for L in layers:
        posn = torch.arange(0, n, device=dev)
        slots = (L.block_tables[0, (posn // BLOCK)].to(torch.int64) * BLOCK + posn % BLOCK).to(torch.int32)
        qsl = torch.tensor([0, n], dtype=torch.int32, device=dev)
        seq = torch.tensor([n], dtype=torch.int32, device=dev)
        batch = ffi.Warp34AttentionBatch(qsl.data_ptr(), None, seq.data_ptr(), L.block_tables.data_ptr(),
                                         slots.data_ptr(), None, None, 1, n, L.max_blocks, n, n, 0, 0, 0.0625, 0)
        per_layer.append((L, slots, batch, qsl, seq))
    vp = lambda t: C.c_void_p(t.data_ptr())

    def step(i):
        L, _, batch, _, _ = per_layer[i % n_layers]
        rc = lib.warp34_kv_cache_write_bf16(C.byref(ex), C.byref(L.layout), C.byref(batch), vp(k), vp(v))
        if rc:
            raise RuntimeError("warp34_kv_cache_write_bf16 rc=%d" % rc)

    condition(args, torch, step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    # algorithmic bytes: one bf16 row read and one encoded row written per (token, kv head, K | V), one slot per token
    bytes_step = n * KV_HEADS * 2 * (HEAD_DIM * 2 + ROW_BYTES[fmt]) + n * 4
    gbs = bytes_step / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "quantize-on-append into %s pages: us/layer + achieved HBM GB/s" % fmt.upper(),
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "us_per_layer": round(ms * 1e3, 2), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "tokens": n, "kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
                   "page_tokens": BLOCK, "kv_format": "tq4+wht256" if fmt == "tq4" else fmt, "kv_pools_cycled": n_layers,
                   "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
                     "kernel": "kv_append_kernel", "avg_launch_us": round(ms * 1e3, 2)},
    }))


def run_producer(args, torch, lib, ffi, layers, n, n_layers, fmt):
    """QK RMSNorm + RoPE over packed bf16 [n, (16 + 2 * 2) * 256] rows with the K / V rows written
    into TQ4 pages: the fused entry point against the two-call sequence (operator in place, then
    the strided append).  One step = one layer's producer work for an n-token chunk."""
    dev = "cuda:0"
    row = (Q_HEADS + 2 * KV_HEADS) * HEAD_DIM
    qkv0 = synth_normal(torch, ffi, (n, row), 11)
    qkv = qkv0.clone()
    q_out = torch.empty((n, Q_HEADS * HEAD_DIM), dtype=torch.bfloat16, device=dev)
    qw = (1.0 + 0.1 * synth_normal(torch, ffi, (HEAD_DIM,), 12, torch.float32)).to(torch.bfloat16)
    kw = (1.0 + 0.1 * synth_normal(torch, ffi, (HEAD_DIM,), 13, torch.float32)).to(torch.bfloat16)
    half = HEAD_DIM // 2
    inv_freq = 1.0 / (10000.0 ** (torch.arange(half, device=dev) / half))
    ang = torch.arange(n, device=dev)[:, None] * inv_freq[None, :]
    table = torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).float().contiguous()
    pos = torch.arange(n, dtype=torch.int32, device=dev)
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, 0, 0, 0)
    per_layer = []
    for L in layers:
        slots = torch.cat(L.tail_slots) if len(L.tail_slots) > 1 else L.tail_slots[0]
        posn = torch.arange(0, n, device=dev)
        slots = (L.block_tables[0, (posn // BLOCK)].to(torch.int64) * BLOCK + posn % BLOCK).to(torch.int32)
        qsl = torch.tensor([0, n], dtype=torch.int32, device=dev)
        seq = torch.tensor([n], dtype=torch.int32, device=dev)
        batch = ffi.Warp34AttentionBatch(qsl.data_ptr(), None, seq.data_ptr(), L.block_tables.data_ptr(),
                                         slots.data_ptr(), None, None, 1, n, L.max_blocks, n, n, 0, 0, 0.0625, 0)
        per_layer.append((L, slots, batch, qsl, seq))
    vp = lambda t: C.c_void_p(t.data_ptr())

    def fused(i):
        L, slots, batch, _, _ = per_layer[i % n_layers]
        rc = lib.warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table(
            C.byref(ex), vp(qkv), vp(q_out), vp(pos), vp(qw), vp(kw), vp(table), C.byref(L.layout), vp(slots),
            n, Q_HEADS, KV_HEADS, HEAD_DIM, n, 1e-6)
        if rc:
            raise RuntimeError("fused producer rc=%d" % rc)

    def two_calls(i):
        L, slots, batch, _, _ = per_layer[i % n_layers]
        rc = lib.warp34_dflash_qk_norm_rope_bf16_f32_table_qout(
            C.byref(ex), vp(qkv), vp(q_out), vp(pos), vp(qw), vp(kw), vp(table), n, Q_HEADS, KV_HEADS, HEAD_DIM, n, 1e-6)
        k_cols = C.c_void_p(qkv.data_ptr() + 2 * Q_HEADS * HEAD_DIM)
        v_cols = C.c_void_p(qkv.data_ptr() + 2 * (Q_HEADS + KV_HEADS) * HEAD_DIM)
        rc = rc or lib.warp34_kv_cache_write_strided_bf16(C.byref(ex), C.byref(L.layout), C.byref(batch), k_cols,
                                                          v_cols, row)
        if rc:
            raise RuntimeError("operator + append rc=%d" % rc)

    def timed(step):
        condition(args, torch, step)
        for i in range(args.warmup):
            step(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.steps):
            step(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms_fused = timed(fused)
    ms_two = timed(two_calls)
    # algorithmic bytes: the packed row is read once, Q is written once, one K and one V row per kv head
    bytes_step = n * (row * 2 + Q_HEADS * HEAD_DIM * 2 + 2 * KV_HEADS * ROW_BYTES[fmt]) + n * HEAD_DIM * 4
    gbs = bytes_step / (ms_fused * 1e-3) / 1e9
    print(json.dumps({
        "metric": "QK RMSNorm + RoPE fused with the %s append: us/layer + achieved HBM GB/s" % fmt.upper(),
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_fused, 6), "us_per_layer": round(ms_fused * 1e3, 2),
        "us_per_layer_operator_then_append": round(ms_two * 1e3, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 arithmetic on bf16 rows, %s rows written" % fmt.upper(), "data": "synthetic",
        "config": {"workload": args.workload, "tokens": n, "q_heads": Q_HEADS, "kv_heads": KV_HEADS,
                   "head_dim": HEAD_DIM, "page_tokens": BLOCK, "kv_format": "tq4+wht256" if fmt == "tq4" else fmt,
                   "kv_pools_cycled": n_layers, "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
                     "kernel": "qk_norm_rope_kernel<true, true> (fused cache write)",
                     "avg_launch_us": round(ms_fused * 1e3, 2)},
    }))


def run_fused_qk_gate(args, torch, lib, ffi, layers, n, n_layers, fmt):
    """The target model's Q/K producer (Gemma RMSNorm + interleaved mRoPE + gate split) over the fp16 rows of
    one fused projection [n, 16 * 512 + 2 * 2 * 256], with the K / V rows written into the pages: the fused
    entry point against the reference's two calls (operator, then the strided append).  One step = one
    layer's producer work for an n-token chunk."""
    dev = "cuda:0"
    qg_w, kv_w = Q_HEADS * 2 * HEAD_DIM, KV_HEADS * HEAD_DIM
    row = qg_w + 2 * kv_w
    proj = synth_normal(torch, ffi, (n, row), 21).to(torch.float16)
    q_out = torch.empty((n, Q_HEADS * HEAD_DIM), dtype=torch.float16, device=dev)
    gate_out = torch.empty_like(q_out)
    k_out = torch.empty((n, kv_w), dtype=torch.float16, device=dev)
    qw = (0.1 * synth_normal(torch, ffi, (HEAD_DIM,), 22, torch.float32)).to(torch.float16)
    kw = (0.1 * synth_normal(torch, ffi, (HEAD_DIM,), 23, torch.float32)).to(torch.float16)
    pos = torch.arange(n, dtype=torch.int32, device=dev).repeat(3, 1).contiguous()
    ex = ffi.Warp34Exec(torch.cuda.current_stream().cuda_stream, 0, 0, 0)
    per_layer = []
    posn = torch.arange(0, n, device=dev)
    for L in layers:
        slots = (L.block_tables[0, (posn // BLOCK)].to(torch.int64) * BLOCK + posn % BLOCK).to(torch.int32)
        qsl = torch.tensor([0, n], dtype=torch.int32, device=dev)
        seq = torch.tensor([n], dtype=torch.int32, device=dev)
        batch = ffi.Warp34AttentionBatch(qsl.data_ptr(), None, seq.data_ptr(), L.block_tables.data_ptr(),
                                         slots.data_ptr(), None, None, 1, n, L.max_blocks, n, n, 0, 0, 0.0625, 0)
        per_layer.append((L, slots, batch, qsl, seq))
    at = lambda off: C.c_void_p(proj.data_ptr() + 2 * off)
    vp = lambda t: C.c_void_p(t.data_ptr())
    rot, mrope, theta, eps = 64, (11, 11, 10), 1.0e7, 1.0e-6

    def fused(i):
        L, slots, _, _, _ = per_layer[i % n_layers]
        rc = lib.warp34_fused_qk_rmsnorm_rope_gate_kv_write_f16(
            C.byref(ex), at(0), at(qg_w), at(qg_w + kv_w), vp(qw), vp(kw), vp(pos), None, vp(q_out), None,
            vp(gate_out), C.byref(L.layout), vp(slots), n, n, Q_HEADS, KV_HEADS, HEAD_DIM, rot, mrope[0], mrope[1],
            mrope[2], row, row, row, theta, eps)
        if rc:
            raise RuntimeError("fused producer rc=%d" % rc)

    def two_calls(i):
        L, slots, batch, _, _ = per_layer[i % n_layers]
        rc = lib.warp34_fused_qk_rmsnorm_rope_gate_strided_f16(
            C.byref(ex), at(0), at(qg_w), vp(qw), vp(kw), vp(pos), None, vp(q_out), vp(k_out), vp(gate_out), n, n,
            Q_HEADS, KV_HEADS, HEAD_DIM, rot, mrope[0], mrope[1], mrope[2], row, row, theta, eps)
        rc = rc or lib.warp34_kv_cache_write_strided(C.byref(ex), C.byref(L.layout), C.byref(batch), vp(k_out),
                                                     at(qg_w + kv_w), kv_w, row)
        if rc:
            raise RuntimeError("operator + append rc=%d" % rc)

    def timed(step):
        condition(args, torch, step)
        for i in range(args.warmup):
            step(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.steps):
            step(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    ms_fused = timed(fused)
    ms_two = timed(two_calls)
    # algorithmic bytes: the projection row is read once, Q and the gate are written once, one K and one V
    # row per kv head go to the pages
    bytes_step = n * (row * 2 + 2 * Q_HEADS * HEAD_DIM * 2 + 2 * KV_HEADS * ROW_BYTES[fmt]) + 3 * n * 4
    gbs = bytes_step / (ms_fused * 1e-3) / 1e9
    print(json.dumps({
        "metric": "Gemma RMSNorm + mRoPE + gate split fused with the %s append: us/layer + achieved HBM GB/s" % fmt.upper(),
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_fused, 6), "us_per_layer": round(ms_fused * 1e3, 2),
        "us_per_layer_operator_then_append": round(ms_two * 1e3, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 arithmetic on fp16 rows, %s rows written" % fmt.upper(), "data": "synthetic",
        "config": {"workload": args.workload, "tokens": n, "q_heads": Q_HEADS, "kv_heads": KV_HEADS,
                   "head_dim": HEAD_DIM, "rotary_dim": rot, "page_tokens": BLOCK,
                   "kv_format": "tq4+wht256" if fmt == "tq4" else fmt, "kv_pools_cycled": n_layers,
                   "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
                     "traffic_source": PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
                     "kernel": "fused_qk_norm_rope_gate_kernel (cache write fused)",
                     "avg_launch_us": round(ms_fused * 1e3, 2)},
    }))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU only (this build has no multi-GPU path); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch

    from warp34_amd import ffi

    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = ffi.load()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.calibrate_copy:
        # plain device copies: scale reference for the traffic counters, and the streaming rate this
        # device reaches on the simplest possible kernel (read + written bytes per second)
        n = 256 << 20
        src = torch.full((n,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 10
        print(json.dumps({"calibrate_copy_bytes": n, "copies": 13,
                          "copy_GBps_read_plus_write": round(2 * n / ms / 1e6, 1)}))
        return
    result = run_workload(args, torch, lib, ffi, dev)
    if result is None:
        return
    if args.workload == "tq4_decode_b1_ctx131072" and not args.ctx and not args.no_batch_point:
        # the same metric with eight 131 072-token sequences in the batch (the fixed costs of a
        # launch amortised): reported beside the headline, never as `value`
        import copy

        sub = copy.copy(args)
        sub.workload, sub.steps, sub.warmup = "tq4_decode_b8_ctx131072", 200, 20
        torch.cuda.empty_cache()
        r8 = run_workload(sub, torch, lib, ffi, dev)
        r8.pop("_sample")
        result["batch_point"] = {"workload": sub.workload, "us_per_layer": r8["us_per_layer"],
                                 "GBps": r8["value"], "frac": r8["roofline"]["frac"], "steps": sub.steps,
                                 "kv_bytes_per_step": r8["config"]["kv_bytes_per_step"]}
    sample = result.pop("_sample")
    if not args.no_cpu_baseline:
        import oracle

        result["cpu_baseline"] = cpu_baseline(torch, sample, min(oracle.hw_threads(), 16))
    print(json.dumps(result))


def condition(args, torch, launch):
    """Device conditioning, before the warm-up steps and outside every timed region: `launch(i)`
    repeated for args.condition_ms of wall time.  A serving loop runs for seconds; a fresh process
    that times 5 + 20 launches of 27 us measures the first millisecond after the pools were filled,
    while the GPU's clock governor is still ramping (same library, same box: one 131 072-token
    sequence 26.0-29.0 us per layer without, 25.4-27.5 with; eight sequences 130 -> 116 us).
    --condition-ms 0 switches it off.  Returns the number of launches."""
    n = 0
    if args.condition_ms > 0:
        t_end = time.perf_counter() + args.condition_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(16):
                launch(n)
                n += 1
            torch.cuda.synchronize()
    return n


def run_workload(args, torch, lib, ffi, dev):
    """Builds the pools of args.workload, times it and returns the result line as a dict
    (None for the prefill workloads, which print their own line)."""
    fmt, ctx, pool_tokens = build_workload(args.workload)
    if args.ctx:
        ctx = np.array([args.ctx], dtype=np.int64)
        args.workload = "%s_decode_b1_ctx%d" % (fmt, args.ctx)
    total_tokens_kv = int(ctx.sum())
    row_bytes = ROW_BYTES[fmt]
    kv_bytes = total_tokens_kv * KV_HEADS * 2 * row_bytes  # algorithmic bytes per step (K + V rows)
    shared = SHARED_PREFIX.get(args.workload, 0)
    pool_pages = max(sum((int(c) + BLOCK - 1) // BLOCK for c in ctx) + 16, pool_tokens // BLOCK)
    pool_pages -= (len(ctx) - 1) * (shared // BLOCK)
    if shared:  # unique bytes: the prefix once, every private suffix once
        kv_bytes = (shared + sum(int(c) - shared for c in ctx)) * KV_HEADS * 2 * row_bytes
    layer_bytes = 2 * pool_pages * KV_HEADS * BLOCK * row_bytes
    n_layers = args.layers or max(2, -(-(640 << 20) // layer_bytes))
    if args.workload.startswith("tq4_append_") and not args.layers:
        n_layers = 8  # the chunk being appended is cache-hot in real use too (its producer has just written it)
    layers = [Layer(torch, lib, ffi, fmt, ctx, pool_pages, s, shared) for s in range(n_layers)]

    if "_prefill_" in args.workload:
        run_prefill(args, torch, lib, ffi, layers, ctx, n_layers, pool_pages, fmt)
        return None
    if args.workload.startswith("attn_output_gate"):
        run_gate(args, torch, lib, ffi)
        return None
    if "_qsa_sparse_" in args.workload:
        run_qsa(args, torch, lib, ffi, layers, int(ctx[0]), n_layers, int(args.workload.split("_")[3].split("x")[0]), fmt)
        return None
    if "_fused_qk_gate_append_" in args.workload:
        run_fused_qk_gate(args, torch, lib, ffi, layers, int(ctx[0]), n_layers, fmt)
        return None
    if "_norm_rope_append_" in args.workload:
        run_producer(args, torch, lib, ffi, layers, int(ctx[0]), n_layers, fmt)
        return None
    if "_append_" in args.workload:
        run_append(args, torch, lib, ffi, layers, int(ctx[0]), n_layers, fmt)
        return None

    R = len(ctx)
    ql = VERIFY_Q.get(args.workload, 1)  # query tokens per request (1 = decode)
    q = synth_normal(torch, ffi, (R * ql, Q_HEADS, HEAD_DIM), 7)
    out = torch.zeros_like(q)
    qsl = (torch.arange(0, R + 1, dtype=torch.int32, device=dev) * ql).to(torch.int32)
    seq = torch.tensor(ctx, dtype=torch.int32, device=dev)
    ctxb = (seq - ql).to(torch.int32)
    # at least 32 MB, and what the library asks for this batch shape
    scratch_bytes = max(32 << 20, int(lib.warp34_paged_attention_scratch_bytes(R * ql, Q_HEADS, int(ctx.max()))))
    scratch = torch.zeros(scratch_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    ex = ffi.Warp34Exec(stream, scratch.data_ptr(), scratch_bytes, 0)
    batches = []
    for L in layers:
        batches.append(ffi.Warp34AttentionBatch(
            qsl.data_ptr(), ctxb.data_ptr(), seq.data_ptr(), L.block_tables.data_ptr(), None, None, None,
            R, R * ql, L.max_blocks, ql, int(ctx.max()), 0, 0, 1.0 / 16.0, 0))

    def step(i):
        L = layers[i % n_layers]
        rc = lib.warp34_paged_attention_bf16(C.byref(ex), C.byref(L.layout), C.byref(batches[i % n_layers]),
                                             C.c_void_p(q.data_ptr()), C.c_void_p(out.data_ptr()), Q_HEADS)
        if rc:
            raise RuntimeError("warp34_paged_attention_bf16 rc=%d" % rc)

    n_cond = condition(args, torch, step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t_wall0 = time.perf_counter()
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    t_wall = time.perf_counter() - t_wall0
    ms_per_step = e0.elapsed_time(e1) / args.steps
    assert torch.isfinite(out.float()).all()
    step(0)  # layer 0 once more: its output is what the CPU leg checks
    torch.cuda.synchronize()
    sample = {"layer": layers[0], "q": q, "ctx": ctx, "ql": ql, "fmt": fmt, "out": out.clone()}

    gbs = kv_bytes / (ms_per_step * 1e-3) / 1e9
    result = {
        "metric": "paged TQ4 decode attn: \u00b5s/layer + achieved HBM GB/s (% peak) at 128K ctx",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "conditioning": {"ms": args.condition_ms, "launches": n_cond,
                         "what": "the same launches, untimed, before the warm-up steps: GPU clocks at their sustained state"},
        "ms_per_step": round(ms_per_step, 6),
        "us_per_layer": round(ms_per_step * 1e3, 3),
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if fmt == "bf16" else "f16",  # type of the MFMA operands; sums and softmax in f32
        "dtype_detail": {"tq4": "f16 MFMA operands (TQ4 codes -> fp16 centroids), f32 accumulate, bf16 Q/out",
                  "bf16": "bf16 MFMA operands, f32 accumulate, bf16 Q/out",
                  "fp8": "f16 MFMA operands (E4M3 codes widened, fp32 block scales), f32 accumulate, bf16 Q/out",
                  "q8_0": "f16 MFMA operands (int8 codes widened, fp32 block scales), f32 accumulate, bf16 Q/out"}[fmt],
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "requests": R, "query_tokens_per_request": ql, "shared_prefix_tokens": shared,
            "context_tokens_total": total_tokens_kv,
            "q_heads": Q_HEADS, "kv_heads": KV_HEADS, "head_dim": HEAD_DIM, "page_tokens": BLOCK,
            "kv_format": "tq4+wht256" if fmt == "tq4" else fmt, "kv_pools_cycled": n_layers,
            "pool_pages": pool_pages,
            "kv_bytes_per_step": kv_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            # HBM bytes per launch as the named profile measured them (rocprofv3 counters cannot be read
            # inside this process): a figure of that profile's run, not of this one; null with --ctx
            "traffic": None if args.ctx else PROFILED_TRAFFIC.get(args.workload, (None, None))[0],
            "traffic_source": None if args.ctx else PROFILED_TRAFFIC.get(args.workload, (None, None))[1],
            "traffic_measured_in_this_run": False,
            "kernel": ("shared_prefix_probe_kernel + paged_prefill_tq4_kernel (shared pages, 32 parts) + "
                       "paged_attn_tq4_kernel (private rest) + split_merge_kernel, all inside the timed launch")
                      if args.workload in SHARED_PREFIX else
                      "paged_attn_%s_kernel (+ merge kernel, both inside the timed launch)"
                      % (("tq4" if fmt == "tq4" else "rows") + ("_balanced" if R > 1 and ql == 1 else "")),
            "avg_launch_us": round(ms_per_step * 1e3, 3),
            "host_wall_us_per_step": round(t_wall / args.steps * 1e6, 2),
        },
    }
    result["_sample"] = sample
    return result


if __name__ == "__main__":
    main()
