#!/usr/bin/env python3
"""Benchmark of the quantized linear-layer path on one MI355X.

Default workload (`decode_q4k_8b_stack`): one decode token's worth of
projections of a Qwen3-8B-shaped decoder with Q4_K weights at M = 1 — 36 layers
x (q, k, v, o, gate, up, down) plus the LM head over 4.26 GB of distinct weight
buffers (far beyond the 256 MB last-level cache, so the weights stream from HBM
every step), called as the reference's attention and MLP blocks call them:
qkv_proj.forward(x) and gate_up_proj.forward(x) are one projection-group call
each (three / two separate weights), o, down and the LM head single calls =
145 calls per step (`--calls per-projection`: 253 single calls).  A step is one
pass over all of them, replayed from a HIP graph.  `value` is algorithmic
bytes (GGUF weight bytes + f32 activations in and out) per second.

Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this build is
single-GPU (the path would shard by output rows without communication).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E peak
BF16_PEAK_TFLOPS = 2500.0    # MI355X published dense bf16 MFMA peak

Q8_0, Q4_K = 8, 12
BPE = {Q8_0: 34 / 32, Q4_K: 144 / 256}

# Qwen3-8B projections: (name, n, k)
LAYER_8B = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
            ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288)]
LM_HEAD_8B = ("lm_head", 151936, 4096)
N_LAYERS_8B = 36


_PROBE = None


def probe():
    """bench_probe/libbench_probe.so: the read-only and copy kernels this benchmark times beside the
    library (built by `make -C bench_probe` / __graft_entry__.build(); not part of libizwi_qmm.so)."""
    global _PROBE
    if _PROBE is None:
        import ctypes as C
        path = os.path.join(ROOT, "bench_probe", "libbench_probe.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `make -C bench_probe`")
        lib = C.CDLL(path)
        lib.bench_probe_stream_read.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p]
        lib.bench_probe_stream_read.restype = C.c_int
        lib.bench_probe_stream_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_void_p]
        lib.bench_probe_stream_copy.restype = C.c_int
        _PROBE = lib
    return _PROBE


def gemv_bytes(dtype, n, k, m):
    return n * k * BPE[dtype] + 4 * m * k + 4 * m * n


def synth_normal(seed, shape, std=1.0, mean=0.0):
    """Seeded N(mean, std) f32 values: the benchmark's own input generator."""
    import numpy as np
    v = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    return (v * np.float32(std) + np.float32(mean)).astype(np.float32)


def quantize_synthetic(dtype, w):
    """GGUF block bytes of a [rows, k] f32 matrix by a plain per-block min / max quantizer (valid Q8_0 /
    Q4_K blocks of the right statistics for a benchmark; not candle's search for the best scales, which no
    timed region depends on)."""
    import numpy as np
    rows, k = w.shape
    if dtype == Q8_0:
        x = w.reshape(-1, 32)
        d = (np.abs(x).max(axis=1) / 127.0).astype(np.float16)
        df = d.astype(np.float32)
        q = np.where(df[:, None] > 0, np.rint(x / np.where(df > 0, df, 1)[:, None]), 0).clip(-127, 127).astype(np.int8)
        out = np.empty((x.shape[0], 34), np.uint8)
        out[:, :2] = d.view(np.uint8).reshape(-1, 2)
        out[:, 2:] = q.view(np.uint8)
        return out.reshape(-1)
    assert dtype == Q4_K and k % 256 == 0
    x = w.reshape(-1, 8, 32)                                  # super-block, sub-block, element
    mn = np.minimum(x.min(axis=2), 0.0)
    scale = (x.max(axis=2) - mn) / 15.0                       # per sub-block
    d = (scale.max(axis=1) / 63.0).astype(np.float16)
    dmin = ((-mn).max(axis=1) / 63.0).astype(np.float16)
    df, dmf = d.astype(np.float32), dmin.astype(np.float32)
    sc = np.where(df[:, None] > 0, np.rint(scale / np.where(df > 0, df, 1)[:, None]), 0).clip(0, 63).astype(np.uint8)
    m = np.where(dmf[:, None] > 0, np.rint(-mn / np.where(dmf > 0, dmf, 1)[:, None]), 0).clip(0, 63).astype(np.uint8)
    step = df[:, None] * sc.astype(np.float32)
    q = np.where(step[:, :, None] > 0, np.rint((x + (dmf[:, None] * m)[:, :, None]) / np.where(step > 0, step, 1)[:, :, None]), 0)
    q = q.clip(0, 15).astype(np.uint8)
    out = np.empty((x.shape[0], 144), np.uint8)
    out[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    out[:, 2:4] = dmin.view(np.uint8).reshape(-1, 2)
    out[:, 4:8] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)       # the 6-bit scales and mins in 12 bytes
    out[:, 8:12] = (m[:, 0:4] & 63) | ((m[:, 4:8] >> 4) << 6)
    out[:, 12:16] = (sc[:, 4:8] & 15) | ((m[:, 4:8] & 15) << 4)
    qq = q.reshape(-1, 4, 2, 32)                              # 64-element pair, low / high nibble, byte
    out[:, 16:] = (qq[:, :, 0, :] | (qq[:, :, 1, :] << 4)).reshape(-1, 128)
    return out.reshape(-1)


def make_blocks(dtype, n, k, seed, pool_rows=None):
    """Seeded N(0, 0.02) weights quantized to GGUF blocks.  For very tall matrices only `pool_rows`
    distinct rows are generated and repeated."""
    import numpy as np
    rows = n if pool_rows is None else min(n, pool_rows)
    blocks = quantize_synthetic(dtype, synth_normal(seed, (rows, k), std=0.02))
    if rows < n:
        per_row = blocks.size // rows
        reps = -(-n // rows)
        blocks = np.tile(blocks.reshape(rows, per_row), (reps, 1))[:n].reshape(-1).copy()
    return blocks


def time_graph(torch, fn, steps, warmup):
    """Captures fn() in a HIP graph and times `steps` replays with events on the
    replay stream.  Returns (ms_per_step, graph)."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        fn()  # warm caches / lazy module loads outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        fn()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(steps):
            graph.replay()
        end.record(stream)
        torch.cuda.synchronize()
    return start.elapsed_time(end) / steps, graph


def time_eager(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def build_decode_weights(torch, qa, dtype, n_layers, with_lm_head):
    """Distinct device buffers for every projection of every layer (same seeded
    byte content per projection kind).  Returns [(QMatMul, n, k)]."""
    gg = qa.GgmlDType(dtype)
    host = {name: make_blocks(dtype, n, k, 1000 + i) for i, (name, n, k) in enumerate(LAYER_8B)}
    weights = []
    for _layer in range(n_layers):
        for name, n, k in LAYER_8B:
            weights.append((qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, host[name], (n, k))), n, k))
    if with_lm_head:
        name, n, k = LM_HEAD_8B
        blocks = make_blocks(dtype, n, k, 2000, pool_rows=16384)
        weights.append((qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, blocks, (n, k))), n, k))
    del host
    return weights


def build_packed_weights(torch, qa, dtype, n_layers):
    """The same stack with q|k|v and gate|up row-concatenated into one weight each, as the
    reference's packed_qmatmul_from_qtensors does where it enables projection grouping:
    4 launches per layer instead of 7, identical weight bytes and outputs."""
    gg = qa.GgmlDType(dtype)
    host = {name: (make_blocks(dtype, n, k, 1000 + i), n, k) for i, (name, n, k) in enumerate(LAYER_8B)}

    def packed(names):
        return qa.packed_qmatmul_from_qtensors([(gg, host[nm][0], (host[nm][1], host[nm][2])) for nm in names])

    weights = []
    for _layer in range(n_layers):
        weights.append((packed(("q", "k", "v")), 4096 + 2 * 1024, 4096))
        weights.append((qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, host["o"][0], (4096, 4096))), 4096, 4096))
        weights.append((packed(("gate", "up")), 2 * 12288, 4096))
        weights.append((qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, host["down"][0], (4096, 12288))), 4096, 12288))
    name, n, k = LM_HEAD_8B
    blocks = make_blocks(dtype, n, k, 2000, pool_rows=16384)
    weights.append((qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, blocks, (n, k))), n, k))
    return weights


def decode_calls(torch, dtype, weights, m):
    """(calls, algorithmic bytes) of one decode step with m activation rows."""
    xs = {k: torch.from_numpy(synth_normal(7 + k, (m, k))).cuda() for k in (4096, 12288)}
    calls, total = [], 0.0
    for mm, n, k in weights:
        calls.append((mm, xs[k], torch.empty((m, n), dtype=torch.float32, device="cuda")))
        total += gemv_bytes(dtype, n, k, m)
    return calls, total


def run_calls(qa, calls):
    """calls: (QMatMul, x, y) single projections or ([QMatMul...], x, [y...]) projection groups."""
    import ctypes as C
    from izwi_amd import capi
    from izwi_amd.qmatmul import _stream_ptr
    L = capi.lib()
    sp = _stream_ptr()
    for mm, x, y in calls:
        if isinstance(mm, (list, tuple)):
            n = len(mm)
            handles = (C.c_void_p * n)(*[p.qtensor._h for p in mm])
            outs = (C.c_void_p * n)(*[t.data_ptr() for t in y])
            rc = L.izwi_qmm_forward_group_f32(handles, n, x.data_ptr(), x.shape[0], outs, capi.DEVICE, sp)
        else:
            rc = L.izwi_qmm_forward_f32(mm.qtensor._h, x.data_ptr(), x.shape[0], y.data_ptr(), capi.DEVICE, sp)
        if rc:
            capi.check(rc)


def grouped_decode_calls(torch, dtype, weights, m):
    """The same projections called the way Qwen3Attention::forward / Qwen3Mlp::forward call
    them (qwen3/core.rs:1599, 1787): qkv_proj.forward(x) and gate_up_proj.forward(x) are one
    call each (three / two separate weights), o and down single calls: 4 calls per layer."""
    xs = {k: torch.from_numpy(synth_normal(7 + k, (m, k))).cuda() for k in (4096, 12288)}
    out = lambda n: torch.empty((m, n), dtype=torch.float32, device="cuda")
    calls, total = [], 0.0
    per_layer = len(LAYER_8B)
    n_layers = (len(weights) - 1) // per_layer
    for layer in range(n_layers):
        w = weights[layer * per_layer:(layer + 1) * per_layer]  # q k v o gate up down
        calls.append(([w[0][0], w[1][0], w[2][0]], xs[4096], [out(w[0][1]), out(w[1][1]), out(w[2][1])]))
        calls.append((w[3][0], xs[4096], out(w[3][1])))
        calls.append(([w[4][0], w[5][0]], xs[4096], [out(w[4][1]), out(w[5][1])]))
        calls.append((w[6][0], xs[12288], out(w[6][1])))
        total += sum(gemv_bytes(dtype, n, k, m) for _, n, k in w)
    mm, n, k = weights[-1]
    calls.append((mm, xs[k], out(n)))
    total += gemv_bytes(dtype, n, k, m)
    return calls, total


def cpu_baseline(oracle, dtype, m, budget_s=12.0):
    """The oracle (C restatement of candle-core's scalar CPU matmul, OpenMP over
    output columns) timed on one layer's seven projections of the same workload."""
    import numpy as np
    mats = []
    for i, (name, n, k) in enumerate(LAYER_8B):
        mats.append((n, k, make_blocks(dtype, n, k, 1000 + i), synth_normal(7 + k, (m, k))))
    layer_bytes = sum(gemv_bytes(dtype, n, k, m) for n, k, _, _ in mats)
    for n, k, b, x in mats[:2]:
        oracle.qmatmul(dtype, x, b, n)  # warm
    passes, t0 = 0, time.perf_counter()
    while True:
        for n, k, b, x in mats:
            oracle.qmatmul(dtype, x, b, n)
        passes += 1
        dt = time.perf_counter() - t0
        if dt > budget_s:
            break
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {
        "value": round(layer_bytes * passes / dt / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{passes} passes over one Qwen3-8B layer's 7 projections (M={m}, "
                  f"{layer_bytes / 1e6:.1f} MB algorithmic bytes per pass), {dt:.1f} s; "
                  "C restatement of candle-core 0.10.2 scalar path, not the Candle binary",
    }


def cpu_baseline_table(oracle, torch, qa):
    """Part of the cpu_baseline leg (the only one that touches the oracle): for every BASELINE
    configuration a bounded sample on which the CPU restatement is timed (all host threads) and the HIP
    path's result is compared with it (max |y - y_ref| / max |y_ref|; dequantization bit for bit).
    The GPU times of the same configurations are the bench's other figures."""
    import numpy as np
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))

    def timed(fn, min_s=0.2):
        fn()
        n, t0 = 0, time.perf_counter()
        while True:
            r = fn()
            n += 1
            dt = time.perf_counter() - t0
            if dt > min_s:
                return dt / n, r

    def rel(y, want):
        return float(np.abs(y.astype(np.float64) - want).max() / max(float(np.abs(want).max()), 1e-30))

    def projection_rows(dtype, shapes, m, seed):
        cpu_s, worst, exact = 0.0, 0.0, True
        gg = qa.GgmlDType(dtype)
        for i, (name, n, k) in enumerate(shapes):
            blocks = make_blocks(dtype, n, k, seed + i)
            x = synth_normal(seed + 50 + k, (m, k))
            dt, want = timed(lambda: oracle.qmatmul(dtype, x, blocks, n), 0.05)
            cpu_s += dt
            qt = qa.QTensor.from_blocks(gg, blocks, (n, k))
            y = qa.QMatMul.from_qtensor(qt).forward(torch.from_numpy(x).cuda()).cpu().numpy()
            worst = max(worst, rel(y, want))
            if i == 0:
                exact = exact and np.array_equal(qt.dequantize().cpu().numpy().view(np.uint32),
                                                 oracle.dequantize(dtype, blocks, n, k).view(np.uint32))
            del qt
        return {"cpu_ms": round(cpu_s * 1e3, 3), "max_rel_err": float(f"{worst:.2e}"), "dequant_bit_exact": bool(exact)}

    table = {"threads": threads}
    table["C1_q8_0_3072x1024_m1"] = projection_rows(Q8_0, [("up", 3072, 1024)], 1, 3100)
    table["C2_q8_0_0p6b_layer"] = {f"m{m}": projection_rows(Q8_0, LAYER_06B, m, 3200) for m in (1, 4, 16, 64)}
    table["C3_q4k_8b_layer"] = {f"m{m}": projection_rows(Q4_K, LAYER_8B, m, 3300) for m in (1, 8, 16)}
    # C4: bf16 activations, prefill kernel; the CPU restatement on one 1024 x 4096 projection at M = 512
    c4 = {}
    for dtype, label in ((Q4_K, "q4k"), (Q8_0, "q8_0")):
        n, k, m = 1024, 4096, 512
        blocks = make_blocks(dtype, n, k, 3400)
        xb = torch.from_numpy(synth_normal(3401, (m, k))).cuda().to(torch.bfloat16)
        xf = xb.float().cpu().numpy()
        dt, want = timed(lambda: oracle.qmatmul(dtype, xf, blocks, n), 0.05)
        y = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k))).forward_bf16_to_f32(xb)
        c4[f"{label}_k_proj_m512"] = {"cpu_ms": round(dt * 1e3, 2), "max_rel_err": float(f"{rel(y.cpu().numpy(), want):.2e}")}
    table["C4_prefill_sample"] = c4
    # C5: the MoE layer; the oracle is scalar per pair, so T = 512 is checked and timed on 16 of its tokens
    e, top_k, hidden, inter = 128, 8, 2048, 768
    gate = np.tile(make_blocks(Q4_K, 8 * inter, hidden, 31), e // 8)
    up = np.tile(make_blocks(Q4_K, 8 * inter, hidden, 32), e // 8)
    down = np.tile(make_blocks(Q4_K, 8 * hidden, inter, 33), e // 8)
    gg = qa.GgmlDType(Q4_K)
    experts = qa.MoeExperts(qa.QTensor.from_blocks(gg, gate, (e, inter, hidden)), qa.QTensor.from_blocks(gg, up, (e, inter, hidden)),
                            qa.QTensor.from_blocks(gg, down, (e, hidden, inter)))
    c5 = {}
    for t in (1, 16, 512):
        x = synth_normal(40 + t, (t, hidden))
        logits = synth_normal(50 + t, (t, e))
        ids, wts = qa.moe_route(torch.from_numpy(logits).cuda(), top_k)
        perm, offsets = qa.moe_sort(ids, e)
        out = experts.forward(torch.from_numpy(x).cuda(), ids, wts, perm, offsets).cpu().numpy()
        want_ids, want_wts = oracle.moe_route(logits, top_k)
        want_perm, want_offsets = oracle.moe_sort(want_ids, e)
        rows = np.arange(t) if t <= 16 else np.linspace(0, t - 1, 16).astype(np.int64)
        t0 = time.perf_counter()
        want = oracle.moe_forward(Q4_K, x[rows], want_ids[rows], want_wts[rows], gate, up, down, e, inter)
        dt = time.perf_counter() - t0
        c5[f"t{t}"] = {"cpu_ms_per_token": round(dt * 1e3 / rows.size, 3), "tokens_timed": int(rows.size),
                       "max_rel_err": float(f"{rel(out[rows], want):.2e}"),
                       "indices_bit_exact": bool(np.array_equal(ids.cpu().numpy(), want_ids)
                                                 and np.array_equal(perm.cpu().numpy(), want_perm)
                                                 and np.array_equal(offsets.cpu().numpy(), want_offsets))}
    table["C5_moe_q4k_30b_a3b"] = c5
    del experts
    torch.cuda.empty_cache()
    return table


def prefill_extra(torch, qa, dtype, m, steps=20, warmup=5, only=None, form=None):
    """TFLOP/s of the prefill kernel per projection and per projection group (extra report, not
    `value`): bf16 activations in HBM, bf16 output, called through the C ABI on preallocated buffers.
    `qkv` and `gate_up` are the calls Qwen3Attention::forward / Qwen3Mlp::forward make (q, k, v resp.
    gate, up on the same activations) as one izwi_qmm_forward_group_bf16 call: one launch.
    `form`: None = the library's default (weights dequantized to bf16 in LDS inside the matmul kernel),
    "plane" = the alternative (one dequantization pass per call into a bf16 plane, then a plain bf16
    matrix-core loop; the pass is inside the timed call)."""
    import ctypes as C
    from izwi_amd import capi
    from izwi_amd.qmatmul import _stream_ptr
    L = capi.lib()
    before = qa.get_prefill_form()
    if form is not None:
        qa.set_prefill_form({"lds": 0, "plane": 1}[form])
    try:
        return _prefill_extra(torch, qa, dtype, m, steps, warmup, only, C, capi, _stream_ptr, L)
    finally:
        qa.set_prefill_form(before)


def library_gemm_extra(torch, m=2048, steps=20, warmup=5):
    """Extra report, NOT a rate of the path: the vendor library's plain bf16 GEMM (torch.matmul, i.e.
    hipBLASLt: no quantized weights, no dequantization anywhere) at the shapes of the prefill figures, on
    the same kind of data (N(0,1) activations, N(0,0.02) weights) and on zeros.  It prices the target:
    with real data the chip is power-limited under bf16 matrix instructions, and what a tuned pure-bf16
    kernel reaches at these shapes on this box is the practical ceiling of any kernel that also has to
    dequantize."""
    out = {}
    for label, n, k in (("gate_up", 24576, 4096), ("down", 4096, 12288), ("qkv", 6144, 4096)):
        x = torch.from_numpy(synth_normal(3, (m, k))).cuda().to(torch.bfloat16)
        w = torch.from_numpy(synth_normal(4, (n, k), std=0.02)).cuda().to(torch.bfloat16)
        y = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        ms = time_eager(torch, lambda: torch.matmul(x, w.t(), out=y), steps, warmup)
        out[label] = round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1)
        if label == "gate_up":
            x.zero_(), w.zero_()
            ms = time_eager(torch, lambda: torch.matmul(x, w.t(), out=y), steps, warmup)
            out["gate_up_all_zero_operands"] = round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1)
        del x, w, y
    torch.cuda.empty_cache()
    out["note"] = ("torch.matmul bf16 (the vendor GEMM library) on plain bf16 matrices of the same shapes; zeros draw "
                   "less power and run at a higher clock; not the path, not `value`")
    return out


def _prefill_extra(torch, qa, dtype, m, steps, warmup, only, C, capi, _stream_ptr, L):
    out = {}
    gg = qa.GgmlDType(dtype)
    shapes = {name: (i, n, k) for i, (name, n, k) in enumerate(LAYER_8B)}
    cases = [("q", ("q",)), ("k", ("k",)), ("gate", ("gate",)), ("down", ("down",)),
             ("qkv", ("q", "k", "v")), ("gate_up", ("gate", "up"))]
    for label, names in cases:
        if only is not None and label != only:
            continue
        k = shapes[names[0]][2]
        mms = [qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(
            gg, make_blocks(dtype, shapes[nm][1], k, 1000 + shapes[nm][0], 4096), (shapes[nm][1], k))) for nm in names]
        x = torch.from_numpy(synth_normal(3, (m, k))).cuda().to(torch.bfloat16)
        ys = [torch.empty((m, shapes[nm][1]), dtype=torch.bfloat16, device="cuda") for nm in names]
        sp = _stream_ptr()
        n = len(names)
        handles = (C.c_void_p * n)(*[mm.qtensor._h for mm in mms])
        outs = (C.c_void_p * n)(*[y.data_ptr() for y in ys])

        def call():
            if n == 1:
                rc = L.izwi_qmm_forward_bf16(handles[0], x.data_ptr(), m, outs[0], capi.OUT_BF16, capi.DEVICE, sp)
            else:
                rc = L.izwi_qmm_forward_group_bf16(handles, n, x.data_ptr(), m, outs, capi.OUT_BF16, capi.DEVICE, sp)
            if rc:
                capi.check(rc)

        ms = time_eager(torch, call, steps, warmup)
        flops = sum(2.0 * m * shapes[nm][1] * k for nm in names)
        out[label] = round(flops / (ms * 1e-3) / 1e12, 2)
        del mms, x, ys
    return out


LAYER_06B = [("q", 2048, 1024), ("k", 1024, 1024), ("v", 1024, 1024), ("o", 1024, 2048),
             ("gate", 3072, 1024), ("up", 3072, 1024), ("down", 1024, 3072)]


def small_configs_extra(torch, qa, steps=20, warmup=3, n_layers=28):
    """Extra report (not `value`): BASELINE configurations 1 and 2, which are parity cases first.
    Config 1: one Q8_0 [3072, 1024] matvec (M = 1), the same weight called back to back in a graph: it is
    3.3 MB and stays in the caches, so this is launch + critical-path time, not an HBM rate.
    Config 2: the seven Q8_0 projections of a Qwen3-0.6B-shaped layer at M = 1 / 4 / 16 / 64, called as the
    reference's blocks call them (q|k|v group, o, gate|up group, down): `hbm` = 28 layers with their own
    buffers in one graph (470 MB of weights per step: they stream from HBM), `hot` = one layer's buffers
    replayed 28 times (17 MB: cache-resident)."""
    gg = qa.GgmlDType(Q8_0)
    out = {}
    mm = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, make_blocks(Q8_0, 3072, 1024, 11), (3072, 1024)))
    x = torch.from_numpy(synth_normal(12, (1, 1024))).cuda()
    y = torch.empty((1, 3072), dtype=torch.float32, device="cuda")
    calls = [(mm, x, y)] * 64
    t, g = time_graph(torch, lambda: run_calls(qa, calls), steps, warmup)
    b = gemv_bytes(Q8_0, 3072, 1024, 1)
    out["config1_q8_0_3072x1024_m1"] = {"us_per_call": round(t * 1e3 / 64, 2), "gbs": round(b / (t * 1e-3 / 64) / 1e9, 1),
                                        "note": "same 3.3 MB weight every call: cache-resident, launch-bound"}
    del g, calls, mm
    host = {name: make_blocks(Q8_0, n, k, 1100 + i) for i, (name, n, k) in enumerate(LAYER_06B)}

    def layer():
        return [(qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(gg, host[name], (n, k))), n, k) for name, n, k in LAYER_06B]
    layers = [layer() for _ in range(n_layers)]
    c2 = {}
    for m in (1, 4, 16, 64):
        xs = {k: torch.from_numpy(synth_normal(7 + k, (m, k))).cuda() for k in (1024, 2048, 3072)}
        outb = lambda n: torch.empty((m, n), dtype=torch.float32, device="cuda")

        def layer_calls(w):
            return [([w[0][0], w[1][0], w[2][0]], xs[1024], [outb(2048), outb(1024), outb(1024)]),
                    (w[3][0], xs[2048], outb(1024)),
                    ([w[4][0], w[5][0]], xs[1024], [outb(3072), outb(3072)]),
                    (w[6][0], xs[3072], outb(1024))]
        layer_bytes = sum(gemv_bytes(Q8_0, n, k, m) for _, n, k in LAYER_06B)
        cold = [c for w in layers for c in layer_calls(w)]
        t, g = time_graph(torch, lambda: run_calls(qa, cold), max(5, steps // 2), warmup)
        del g
        hot = layer_calls(layers[0]) * n_layers
        th, g = time_graph(torch, lambda: run_calls(qa, hot), max(5, steps // 2), warmup)
        del g
        c2[f"m{m}"] = {"hbm_us_per_layer": round(t * 1e3 / n_layers, 2),
                       "hbm_gbs": round(layer_bytes * n_layers / (t * 1e-3) / 1e9, 1),
                       "hot_us_per_layer": round(th * 1e3 / n_layers, 2),
                       "pct_of_hbm_peak": round(100.0 * layer_bytes * n_layers / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 1)}
    out["config2_q8_0_0p6b_layer"] = c2
    return out


def batched_percall(torch, qa, dtype, m, steps=30, warmup=5):
    """Profiling aid (--batched-percall): microseconds per call of the four projection calls of a
    Qwen3-8B layer at `m` rows on activation records (the matmul launch alone), each kind as a graph of
    36 layers' distinct weights."""
    weights = build_decode_weights(torch, qa, dtype, N_LAYERS_8B, False)
    per = len(LAYER_8B)
    xs = {k: torch.from_numpy(synth_normal(7 + k, (m, k))).cuda() for k in (4096, 12288)}
    recs = {k: qa.ActivationRecords.quantize(qa.GgmlDType(dtype), xs[k]) for k in xs}
    kinds = {"qkv": ([0, 1, 2], 4096), "o": ([3], 4096), "gate_up": ([4, 5], 4096), "down": ([6], 12288)}
    res = {}
    for name, (idx, k) in kinds.items():
        groups = []
        for layer in range(N_LAYERS_8B):
            w = weights[layer * per:(layer + 1) * per]
            groups.append(([w[i][0] for i in idx],
                           [torch.empty((m, w[i][1]), dtype=torch.float32, device="cuda") for i in idx]))

        def fn():
            for ps, outs in groups:
                recs[k].forward_group(ps, outs)
        ms, g = time_graph(torch, fn, steps, warmup)
        res[name] = round(ms * 1e3 / N_LAYERS_8B, 2)
        del g
    res["layer"] = round(sum(res.values()), 2)
    return res


def overlap_what_if_extra(torch, qa, calls, total_bytes, n_streams=3, steps=20, warmup=3):
    """Extra report, NOT a rate of the path: the headline's launches spread round-robin over several
    streams inside the graph, so that a launch starts while its predecessor still runs.  That is only
    legal here because the synthetic calls do not feed each other; in the model they form a chain.  It
    shows what the gaps between dependent launches and their ramp-up cost: the room a dependency-aware
    overlap (the next launch's weight stream started early) could recover."""
    streams = [torch.cuda.Stream() for _ in range(n_streams)]

    def run():
        cur = torch.cuda.current_stream()
        fork = torch.cuda.Event()
        fork.record(cur)
        for s in streams:
            s.wait_event(fork)
        for i, c in enumerate(calls):
            with torch.cuda.stream(streams[i % n_streams]):
                run_calls(qa, [c])
        for s in streams:
            join = torch.cuda.Event()
            join.record(s)
            cur.wait_event(join)
    ms, g = time_graph(torch, run, steps, warmup)
    del g
    return {"gbs": round(total_bytes / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4), "streams": n_streams,
            "note": "launches overlapped as if independent; not the model's dependent chain, not `value`"}


def chained_extra(torch, qa, calls, total_bytes, steps=20, warmup=3):
    """Extra report (not `value`): the headline's dependent calls as ONE launch (izwi_qmm_chain_*: a
    resident grid walks through the steps, hand-over through write-through stores and counters, the
    next step's weights requested before the wait); the LM head behind it as its own call.  Also a
    144-step chain of the smallest projection alone, whose per-step time is the cost of one
    grid-wide hand-over (its 9.4 MB stream in 1.2 us)."""
    def as_step(c):
        mm, x, y = c
        return (list(mm), x, list(y)) if isinstance(mm, (list, tuple)) else ([mm], x, [y])
    chain = qa.DecodeChain([as_step(c) for c in calls[:-1]])

    def run():
        chain.run()
        run_calls(qa, calls[-1:])
    ms, g = time_graph(torch, run, steps, warmup)
    chain.status()
    del g
    small = [as_step(c) for c in calls[1:-1:4]]       # the o projections
    chain_o = qa.DecodeChain(small)
    ms_o, g = time_graph(torch, chain_o.run, steps, warmup)
    chain_o.status()
    del g
    ms_o_calls, g = time_graph(torch, lambda: run_calls(qa, calls[1:-1:4]), steps, warmup)
    del g
    return {"gbs": round(total_bytes / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4), "launches_per_step": 2,
            "us_per_dependent_step_4096x4096_chained": round(ms_o * 1e3 / len(small), 2),
            "us_per_dependent_step_4096x4096_separate_calls": round(ms_o_calls * 1e3 / len(small), 2),
            "note": "one resident kernel for the 144 dependent projection steps + the LM head call; not `value`"}


def records_path_extra(torch, qa, dtype, weights, m, steps=10, warmup=3):
    """Extra report (not `value`): the headline stack at m rows where the projections whose activations
    come out of an RMSNorm (q|k|v, gate|up, LM head) or out of silu(gate) * up (down) are handed
    activation records by that producer (izwi_rms_norm_quantize_records_f32 /
    izwi_qmm_silu_mul_quantize_records_f32) instead of launching a quantizer of their own; o (fed by
    the attention) keeps its quantizer launch.  The producers are not projections and are timed beside
    the stack: one launch each, in place of the norm / elementwise launch the layer has anyway."""
    import ctypes as C
    from izwi_amd import capi
    L = capi.lib()
    gd = qa.GgmlDType(dtype)
    xs = {k: torch.from_numpy(synth_normal(7 + k, (m, k))).cuda() for k in (4096, 12288)}
    recs = {k: qa.ActivationRecords.quantize(gd, xs[k]) for k in (4096, 12288)}
    out = lambda n: torch.empty((m, n), dtype=torch.float32, device="cuda")  # noqa: E731
    per_layer = len(LAYER_8B)
    n_layers = (len(weights) - 1) // per_layer
    plan, total = [], 0.0
    for layer in range(n_layers):
        w = weights[layer * per_layer:(layer + 1) * per_layer]  # q k v o gate up down
        plan.append(("rec", [w[0][0], w[1][0], w[2][0]], recs[4096], [out(w[0][1]), out(w[1][1]), out(w[2][1])]))
        plan.append(("x", w[3][0], xs[4096], out(w[3][1])))
        plan.append(("rec", [w[4][0], w[5][0]], recs[4096], [out(w[4][1]), out(w[5][1])]))
        plan.append(("rec", [w[6][0]], recs[12288], [out(w[6][1])]))
        total += sum(gemv_bytes(dtype, n, k, m) for _, n, k in w)
    mm, n, k = weights[-1]
    plan.append(("rec", [mm], recs[k], [out(n)]))
    total += gemv_bytes(dtype, n, k, m)
    prepared = []
    for kind, mms, src, ys in plan:
        if kind == "rec":
            nn = len(mms)
            prepared.append((kind, (C.c_void_p * nn)(*[p.qtensor._h for p in mms]), nn, src.data.data_ptr(),
                             (C.c_void_p * nn)(*[y.data_ptr() for y in ys])))
        else:
            prepared.append((kind, mms.qtensor._h, 1, src.data_ptr(), ys.data_ptr()))

    def run():
        sp = torch.cuda.current_stream().cuda_stream   # (the capturing stream)
        for kind, h, nn, src, ys in prepared:
            if kind == "rec":
                rc = L.izwi_qmm_forward_group_records_f32(h, nn, src, m, ys, sp)
            else:
                rc = L.izwi_qmm_forward_f32(h, src, m, ys, capi.DEVICE, sp)
            if rc:
                capi.check(rc)
    ms, g = time_graph(torch, run, steps, warmup)
    del g
    # the producers, per call, against the launches they replace
    nw = torch.ones(4096, device="cuda")
    gate = torch.from_numpy(synth_normal(5, (m, 12288))).cuda()
    up = torch.from_numpy(synth_normal(6, (m, 12288))).cuda()
    ynorm = torch.empty_like(xs[4096])
    prod = {}
    for name, fn in (("rms_norm_to_records_4096", lambda sp: L.izwi_rms_norm_quantize_records_f32(
                         int(dtype), xs[4096].data_ptr(), nw.data_ptr(), m, 4096, 1e-6, recs[4096].data.data_ptr(), sp)),
                     ("rms_norm_alone_4096", lambda sp: L.izwi_rms_norm_f32(xs[4096].data_ptr(), nw.data_ptr(), m, 4096, 1e-6,
                                                                         ynorm.data_ptr(), capi.DEVICE, sp)),
                     ("quantizer_alone_4096", lambda sp: L.izwi_qmm_quantize_records_f32(
                         int(dtype), xs[4096].data_ptr(), m, 4096, recs[4096].data.data_ptr(), sp)),
                     ("silu_mul_to_records_12288", lambda sp: L.izwi_qmm_silu_mul_quantize_records_f32(
                         int(dtype), gate.data_ptr(), up.data_ptr(), m, 12288, recs[12288].data.data_ptr(), sp))):
        def many(fn=fn):
            sp = torch.cuda.current_stream().cuda_stream
            for _ in range(32):
                fn(sp)
        t, g = time_graph(torch, many, steps, warmup)
        prod[name + "_us"] = round(t * 1e3 / 32, 2)
        del g
    return {"gbs": round(total / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4), "m": m, "launches_per_step": 145 + n_layers,
            "producers": prod,
            "note": "q|k|v, gate|up, down, LM head read records written by their producers; o quantizes itself; not `value`"}


def host_pointer_extra(qa, weights, m, passes=2):
    """Extra report (not `value`): the same projections called one by one with HOST pointers, the literal
    form of the reference's CPU call (activations in host memory in, results in host memory out): every
    call stages x to the device, runs the kernel, copies y back and waits.  Wall clock, PCIe included."""
    import time
    import numpy as np
    from izwi_amd import capi
    L = capi.lib()
    bufs = [(mm, np.random.default_rng(1).standard_normal((m, k)).astype(np.float32), np.empty((m, n), np.float32))
            for mm, n, k in weights]
    total = sum(mm.qtensor.storage_size_in_bytes() + 4 * m * k + 4 * m * n for mm, n, k in weights)

    def one_pass():
        for mm, x, y in bufs:
            rc = L.izwi_qmm_forward_f32(mm.qtensor._h, x.ctypes.data, m, y.ctypes.data, capi.HOST, None)
            if rc:
                capi.check(rc)
    one_pass()
    t0 = time.perf_counter()
    for _ in range(passes):
        one_pass()
    dt = (time.perf_counter() - t0) / passes
    return {"gbs": round(total / dt / 1e9, 1), "ms_per_step": round(dt * 1e3, 3), "calls_per_step": len(bufs),
            "us_per_call": round(dt * 1e6 / len(bufs), 1)}


def hbm_ceiling_extra(torch, gib=2, reps=10):
    """Extra report: what plain streaming kernels reach on this GPU, beside the nominal 8 TB/s the roofline
    is priced against, `gib` GiB per pass (far beyond the caches): this benchmark's own read-only kernel
    (the decode kernel's load shape: one 768-thread workgroup per CU, nine 16-byte non-temporal loads per
    lane in flight) and its copy kernel (bytes read + written, best of a few grid sizes), and for
    comparison the runtime's device-to-device copy and torch's copy / reduction kernels."""
    n = gib * (1 << 30) // 4
    x = torch.ones(n, dtype=torch.float32, device="cuda")
    y = torch.empty_like(x)
    P = probe()
    sp = torch.cuda.current_stream().cuda_stream

    def checked(rc):
        if rc:
            raise RuntimeError(f"bench_probe call failed: hipError {rc}")
    read_ms = time_eager(torch, lambda: checked(P.bench_probe_stream_read(x.data_ptr(), n * 4, sp)), reps, 2)
    copy_ms = min(time_eager(torch, lambda: checked(P.bench_probe_stream_copy(x.data_ptr(), y.data_ptr(), n * 4, w, sp)), reps, 2)
                  for w in (2, 4, 8))
    out = {"read_gbs": round(n * 4 / (read_ms * 1e-3) / 1e9, 1), "copy_gbs": round(2 * n * 4 / (copy_ms * 1e-3) / 1e9, 1),
           "gib": gib, "kernels": "bench_probe_stream_read / bench_probe_stream_copy (this benchmark's own)"}
    t_copy = time_eager(torch, lambda: y.copy_(x), reps, 2)
    t_read = time_eager(torch, lambda: x.sum(), reps, 2)
    out["torch_copy_gbs"] = round(2 * n * 4 / (t_copy * 1e-3) / 1e9, 1)
    out["torch_sum_read_gbs"] = round(n * 4 / (t_read * 1e-3) / 1e9, 1)
    try:  # the runtime's own device-to-device copy
        import ctypes as C
        hip = C.CDLL("libamdhip64.so")
        hip.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        ms = time_eager(torch, lambda: hip.hipMemcpyAsync(y.data_ptr(), x.data_ptr(), n * 4, 3, sp), reps, 2)
        out["hip_memcpy_d2d_gbs"] = round(2 * n * 4 / (ms * 1e-3) / 1e9, 1)
    except OSError:
        pass
    del x, y
    torch.cuda.empty_cache()
    return out


def read_only_floor_extra(torch, qa, dtype, weights, m, steps=10, warmup=3):
    """Extra report (not `value`): the same step with every launch replaced by a launch that only
    READS as many bytes (bench_probe_stream_read over its own buffers, one per call of the
    headline structure: q|k|v, o, gate|up, down per layer + LM head; distinct buffers, one graph,
    the same dependent chain of 145 launches).  What plain reads of the same bytes in the same
    launches reach on this GPU: the headline is to be read against it as well as against the nominal
    peak."""
    P = probe()
    per_layer = len(LAYER_8B)
    n_layers = (len(weights) - 1) // per_layer
    kinds = ([0, 1, 2], [3], [4, 5], [6])
    sizes = []
    for layer in range(n_layers):
        w = weights[layer * per_layer:(layer + 1) * per_layer]
        for idx in kinds:
            sizes.append(int(sum(gemv_bytes(dtype, w[i][1], w[i][2], m) for i in idx)))
    sizes.append(int(gemv_bytes(dtype, weights[-1][1], weights[-1][2], m)))
    bufs = [torch.randint(0, 255, ((sz + 15) // 16 * 16,), dtype=torch.uint8, device="cuda") for sz in sizes]

    def run():
        sp = torch.cuda.current_stream().cuda_stream
        for b in bufs:
            rc = P.bench_probe_stream_read(b.data_ptr(), b.numel(), sp)
            if rc:
                raise RuntimeError(f"bench_probe_stream_read failed: hipError {rc}")

    t, g = time_graph(torch, run, steps, warmup)
    total = float(sum(sizes))
    out = {"gbs": round(total / (t * 1e-3) / 1e9, 1), "ms_per_step": round(t, 4), "launches_per_step": len(bufs),
           "note": "read-only launches of the same sizes in the same dependent chain; not `value`"}
    del g, bufs
    torch.cuda.empty_cache()
    return out


def neighbours_extra(torch, qa, steps=10, warmup=3):
    """Extra report (not `value`): the decode-step neighbours at Qwen3-8B shapes (32 query heads on
    8 kv heads, head_dim 128, hidden 4096, f32): microseconds per call in a HIP-graph replay and, for
    attention, KV-cache bytes (K and V read once) over time."""
    heads, kvh, d, hidden = 32, 8, 128, 4096
    out = {}
    q = torch.randn(1, heads, 1, d, device="cuda")
    for kv_len in (512, 4096, 32768):
        n_caches = max(2, min(16, (1 << 29) // (kv_len * kvh * d * 8)))  # rotate caches: none stays in L2
        ks = [torch.randn(1, kvh, kv_len, d, device="cuda") for _ in range(n_caches)]
        vs = [torch.randn_like(k) for k in ks]
        reps = max(1, 32 // n_caches)

        def run():
            for _ in range(reps):
                for k, v in zip(ks, vs):
                    qa.try_fused_decode_gqa_attention(q, k, v, heads, kvh, d, d ** -0.5)
        ms, g = time_graph(torch, run, steps, warmup)
        us = ms * 1e3 / (reps * n_caches)
        out[f"attention_kv{kv_len}"] = {"us": round(us, 2), "gbs": round(2 * kvh * kv_len * d * 4 / us / 1e3, 1)}
        del ks, vs, g
    x, w = torch.randn(1, hidden, device="cuda"), torch.randn(hidden, device="cuda")
    qq, kk = torch.randn(1, 1, heads, d, device="cuda"), torch.randn(1, 1, kvh, d, device="cuda")
    qkw, cs = torch.randn(2 * d, device="cuda"), torch.randn(1, d, device="cuda")
    for name, fn in (("rms_norm_1x4096", lambda: qa.try_fused_rms_norm(x, w, 1e-6)),
                     ("qk_rms_norm_40x128", lambda: qa.try_fused_qk_rms_norm(qq, kk, qkw, 1e-6)),
                     ("rope_40x128", lambda: qa.try_fused_rope_pair_bshd(qq, kk, cs))):
        def run():
            for _ in range(64):
                fn()
        ms, g = time_graph(torch, run, steps, warmup)
        out[name] = {"us": round(ms * 1e3 / 64, 2)}
        del g
    torch.cuda.empty_cache()
    return out


def fused_and_q6k_extra(torch, qa, steps=10, warmup=3):
    """Extra report (not `value`): (a) the o / down projections of the 8B stack with bf16 activations in,
    residual added, bf16 out in one call each (izwi_qmm_forward_fused) against the same projections
    as f32 calls with torch's cast / add / cast kernels around them; (b) Q6_K projections of a
    Q4_K_M file (ffn_down, attn_v, output) at M = 1: microseconds and Q6_K bytes over time, and their
    prefill rate at M = 2048 and 512."""
    import numpy as np
    out = {}
    rng = np.random.default_rng(5)

    def q6k(n, k):
        rows = min(n, 2048)
        b = rng.integers(0, 256, size=(rows * k // 256, 210), dtype=np.uint8)
        b[:, 208:210] = (1e-3 * rng.uniform(0.5, 2.0, size=b.shape[0])).astype(np.float16).view(np.uint8).reshape(-1, 2)
        b = np.tile(b.reshape(rows, -1), ((n + rows - 1) // rows, 1))[:n]
        return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, b.reshape(-1), (n, k)))

    for name, n, k, copies in (("ffn_down", 4096, 12288, 8), ("attn_v", 1024, 4096, 16), ("output", 151936, 4096, 2)):
        ws = [q6k(n, k) for _ in range(copies)]
        x = torch.randn(1, k, device="cuda")
        reps = max(1, 32 // copies)

        def run():
            for _ in range(reps):
                for w in ws:
                    w.forward(x)
        ms, g = time_graph(torch, run, steps, warmup)
        us = ms * 1e3 / (reps * copies)
        out[f"q6k_m1_{name}"] = {"us": round(us, 2), "gbs": round(n * k // 256 * 210 / us / 1e3, 1)}
        if name != "output":  # prefill of the same tensor: bf16 in, bf16 out, TFLOP/s
            for m in (2048, 512):
                xb = torch.randn(m, k, device="cuda").bfloat16()
                ms = time_eager(torch, lambda: ws[0].forward(xb), 20, 5)
                out[f"q6k_prefill_tflops_m{m}_{name}"] = round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1)
                del xb
        del ws, g
        torch.cuda.empty_cache()
    mats = []
    for i in range(8):
        mats.append(tuple(qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(
            qa.GgmlDType.Q4K, make_blocks(Q4_K, 4096, k, 1003 if k == 4096 else 1006), (4096, k))) for k in (4096, 12288)))
    xa, xh = torch.randn(1, 4096, device="cuda").bfloat16(), torch.randn(1, 12288, device="cuda").bfloat16()
    res = torch.randn(1, 4096, device="cuda").bfloat16()

    passes = 8  # 64 layers' worth of calls per graph replay, so that the replay's own start-up does not show

    def fused():
        for _ in range(passes):
            for o, dn in mats:
                o.forward_fused(xa, residual=res, out=res)
                dn.forward_fused(xh, residual=res, out=res)

    def unfused():
        r = res
        for _ in range(passes):
            for o, dn in mats:
                r = r + o.forward(xa.float()).bfloat16()
                r = r + dn.forward(xh.float()).bfloat16()

    def plain_f32():  # the same projections as plain f32 calls, nothing around them
        xa32, xh32 = xa.float(), xh.float()
        for _ in range(passes):
            for o, dn in mats:
                o.forward(xa32)
                dn.forward(xh32)
    for name, fn in (("fused", fused), ("unfused", unfused), ("plain_f32_calls_only", plain_f32)):
        ms, g = time_graph(torch, fn, steps, warmup)
        out[f"o_down_bf16_residual_{name}_us_per_layer"] = round(ms * 1e3 / (passes * len(mats)), 2)
        del g
    del mats
    torch.cuda.empty_cache()
    return out


def layer_stack_extra(torch, qa, dtype, steps=10, warmup=3):
    """Extra report (not `value`): one whole decode step of the Qwen3-8B stack composed from the library's
    calls (izwi_amd.qwen3_layer.Qwen3DecodeLayer: q|k|v group and gate/up with their RMSNorm and the
    activation folded in, attention with q/k norm + rotary + cache append inside its launch and the merge
    of its splits, o and down with the residual folded in), from the embedding row of the previous token (read from the
    quantized table) to the final norm folded into the LM head and the greedy argmax: every replay consumes the token
    the one before produced.  f32 activations, HIP-graph replay, at several context lengths."""
    from izwi_amd.qwen3_layer import Qwen3DecodeLayer
    heads, kvh, d, hidden = 32, 8, 128, 4096
    weights = build_decode_weights(torch, qa, dtype, N_LAYERS_8B, True)
    per = len(LAYER_8B)
    ones = lambda n: torch.ones(n, device="cuda")  # noqa: E731
    layers = []
    for i in range(N_LAYERS_8B):
        q, k, v, o, gate, up, down = [w[0] for w in weights[i * per:(i + 1) * per]]
        layers.append(Qwen3DecodeLayer(ones(hidden), ones(hidden), q, k, v, ones(2 * d), o, gate, up, down, heads, kvh, d))
    lm_head, final_norm = weights[-1][0], ones(hidden)
    # token in, token out, all on the device: the step starts with the embedding row of the token the
    # previous step's argmax left (the table is the LM head's quantized matrix, as in a tied checkpoint)
    embed = qa.QuantizedEmbedding(lm_head.qtensor)
    token = torch.zeros(1, dtype=torch.int32, device="cuda")
    cos_sin = torch.randn(1, d, device="cuda")
    out = {}
    for kv_len in (256, 4096):
        caches = [(torch.randn(1, kvh, kv_len, d, device="cuda") * 0.1, torch.randn(1, kvh, kv_len, d, device="cuda") * 0.1)
                  for _ in range(N_LAYERS_8B)]

        def step():
            x = embed.forward(token)
            for layer, (kc, vc) in zip(layers, caches):
                x = layer.forward(x, cos_sin, kc, vc, kv_len - 1)
            token.copy_(qa.argmax(lm_head.forward_normed(x, final_norm, 1e-6)))  # final norm + LM head, greedy next token
        ms, g = time_graph(torch, step, steps, warmup)
        out[f"kv{kv_len}"] = {"ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1)}
        del caches, g
        torch.cuda.empty_cache()
    out["launches_per_token"] = N_LAYERS_8B * 6 + 5  # embedding row, LM head with the norm, two for the argmax, the token copy
    del layers, weights
    torch.cuda.empty_cache()
    return out


def q4_k_m_mix_extra(torch, qa, m=1, steps=20, warmup=3):
    """Extra report (not `value`): the decode stack with the tensor types of a Q4_K_M file of Qwen3-8B (the
    reference's default chat model): attn_v and ffn_down are Q6_K in half of the layers (the first and last
    eighth and every third layer between, as llama.cpp's Q4_K_M recipe picks them) and so is the output
    matrix; everything else is Q4_K.  Q6_K weights are random block bytes with a finite scale.  Same call
    structure as the headline; a q|k|v group with a Q6_K member is split by type inside the library (q|k
    as one launch, v as another)."""
    import numpy as np
    rng = np.random.default_rng(11)

    def q6k_blocks(n, k):
        rows = min(n, 2048)
        b = rng.integers(0, 256, size=(rows * k // 256, 210), dtype=np.uint8)
        b[:, 208:210] = (1e-3 * rng.uniform(0.5, 2.0, size=b.shape[0])).astype(np.float16).view(np.uint8).reshape(-1, 2)
        return np.tile(b.reshape(rows, -1), ((n + rows - 1) // rows, 1))[:n].reshape(-1)

    def more_bits(i, n):
        return i < n // 8 or i >= 7 * n // 8 or (i - n // 8) % 3 == 2
    q4 = {name: make_blocks(Q4_K, n, k, 1000 + i) for i, (name, n, k) in enumerate(LAYER_8B)}
    q6 = {name: q6k_blocks(n, k) for name, n, k in LAYER_8B if name in ("v", "down")}
    shape = {name: (n, k) for name, n, k in LAYER_8B}
    bytes_per = {Q4_K: 144, 14: 210}
    xs = {k: torch.randn(m, k, device="cuda") for k in (4096, 12288)}
    out = lambda n: torch.empty((m, n), dtype=torch.float32, device="cuda")  # noqa: E731
    calls, total, n_q6 = [], 0.0, 0
    for layer in range(N_LAYERS_8B):
        w = {}
        for name, (n, k) in shape.items():
            six = name in q6 and more_bits(layer, N_LAYERS_8B)
            n_q6 += six
            dt = 14 if six else Q4_K
            w[name] = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dt), q6[name] if six else q4[name], (n, k)))
            total += n * k // 256 * bytes_per[dt] + 4 * m * k + 4 * m * n
        calls.append(([w["q"], w["k"], w["v"]], xs[4096], [out(4096), out(1024), out(1024)]))
        calls.append((w["o"], xs[4096], out(4096)))
        calls.append(([w["gate"], w["up"]], xs[4096], [out(12288), out(12288)]))
        calls.append((w["down"], xs[12288], out(4096)))
    name, n, k = LM_HEAD_8B
    head = qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType.Q6K, q6k_blocks(n, k), (n, k)))
    calls.append((head, xs[k], out(n)))
    total += n * k // 256 * 210 + 4 * m * k + 4 * m * n
    ms, g = time_graph(torch, lambda: run_calls(qa, calls), steps, warmup)
    res = {"gbs": round(total / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4), "m": m, "calls_per_step": len(calls),
           "q6k_tensors": n_q6 + 1, "gb_per_step": round(total / 1e9, 3)}
    del calls, g
    torch.cuda.empty_cache()
    return res


def moe_extra(torch, qa, steps=20, warmup=3, layers=8, stacks=4):
    """One MoE layer (route + sort + grouped expert MLP + combine) at the Qwen3-30B-A3B shape: 128
    experts, top-8, hidden 2048, expert intermediate 768, Q4_K; as one call (izwi_moe_layer_f32) and as
    the three calls it is composed of.  Timed as a HIP graph of `layers` consecutive layer calls that
    cycle over `stacks` different sets of expert weights (as the layers of a model follow each other),
    per layer; `us_single_call_graph` is the old figure, a graph that holds one call (it carries the
    replay's own start-up)."""
    import numpy as np
    e, top_k, hidden, inter = 128, 8, 2048, 768
    gg = qa.GgmlDType(Q4_K)

    def stack(n, k, seed):
        one = make_blocks(Q4_K, 8 * n, k, seed)  # 8 distinct experts, repeated
        return qa.QTensor.from_blocks(gg, np.tile(one, e // 8), (e, n, k))

    experts = [qa.MoeExperts(stack(inter, hidden, 31 + 10 * i), stack(inter, hidden, 32 + 10 * i),
                             stack(hidden, inter, 33 + 10 * i)) for i in range(stacks)]
    out = {}
    expert_bytes = 3 * inter * hidden * BPE[Q4_K]
    for t in (1, 16, 512):
        x = torch.from_numpy(synth_normal(40 + t, (t, hidden))).cuda()
        logits = [torch.from_numpy(synth_normal(50 + t + 7 * i, (t, e))).cuda() for i in range(layers)]

        def three_calls():
            for i in range(layers):
                ids, wts = qa.moe_route(logits[i], top_k)
                perm, offsets = qa.moe_sort(ids, e)
                experts[i % stacks].forward(x, ids, wts, perm, offsets)

        def one_call():
            for i in range(layers):
                experts[i % stacks].layer(logits[i], x, top_k)

        ms3, g3 = time_graph(torch, three_calls, steps, warmup)
        del g3
        ms, g = time_graph(torch, one_call, steps, warmup)
        del g
        ms1, g = time_graph(torch, lambda: experts[0].layer(logits[0], x, top_k), steps, warmup)
        del g
        us = ms * 1e3 / layers
        distinct = 0
        for i in range(layers):  # the library's own routing: which experts the tokens touch
            ids_d, _ = qa.moe_route(logits[i], top_k)
            distinct += len(set(ids_d.cpu().numpy().reshape(-1).tolist()))
        distinct /= layers
        rec = {"us": round(us, 1), "us_route_sort_forward_as_three_calls": round(ms3 * 1e3 / layers, 1),
               "us_single_call_graph": round(ms1 * 1e3, 1), "distinct_experts": round(distinct, 1)}
        # algorithmic bytes: the distinct experts' weights + x in + out; flops: 3 matmuls per pair
        rec["gbs"] = round((distinct * expert_bytes + 2 * t * hidden * 4) / us / 1e3, 1)
        rec["tflops"] = round(2.0 * t * top_k * 3 * hidden * inter / us / 1e6, 2)
        out[f"t{t}"] = rec
    return out


def measured_traffic(workload, m, avg_algorithmic):
    """HBM bytes per launch of the decode kernel from the committed rocprofv3 --pmc
    summary (profiles/decode_traffic.json: FETCH_SIZE and WRITE_SIZE per dispatch, each
    scaled by the same counter's reading for a 1 GiB copy).  None when no summary
    matches this workload."""
    path = os.path.join(ROOT, "profiles", "decode_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f).get(f"{workload}:m={m}")
    except (OSError, ValueError):
        return None
    if not rec:
        return None
    return {"bytes_per_launch": rec["bytes_per_launch"],
            "vs_algorithmic": round(rec["bytes_per_launch"] / avg_algorithmic, 3),
            "source": "profiles/decode_traffic.json"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode_q4k_8b_stack",
                    choices=["decode_q4k_8b_stack", "decode_q8_0_8b_stack"])
    ap.add_argument("--m", type=int, default=1, help="activation rows per call (decode batch)")
    ap.add_argument("--layers", type=int, default=N_LAYERS_8B)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (a known-size kernel that scales "
                         "the rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--calls", default="grouped", choices=["grouped", "per-projection"],
                    help="grouped: qkv_proj.forward(x) and gate_up_proj.forward(x) are one call each, as "
                         "the reference's attention and MLP blocks make them (4 calls per layer); "
                         "per-projection: seven izwi_qmm_forward_f32 calls per layer")
    ap.add_argument("--neighbours-only", action="store_true",
                    help="time only the decode-step neighbours (norms, rotary, attention) and print them: for profiling")
    ap.add_argument("--moe-only", action="store_true",
                    help="profiling aid: run only izwi_moe_layer_f32 at the Qwen3-30B-A3B shape with --m tokens "
                         "(--steps calls, eager) and print the time per call, nothing else")
    ap.add_argument("--batched-percall", action="store_true",
                    help="profiling aid: time only the four projection calls of an 8B layer at --m rows (3..64) on "
                         "activation records, per call, and print them")
    ap.add_argument("--prefill-form", default=None, choices=["lds", "plane"],
                    help="with --prefill-only: the form of the prefill product (default: the library's own choice)")
    ap.add_argument("--prefill-only", default=None, choices=["q", "k", "gate", "down", "qkv", "gate_up"],
                    help="profiling aid: run only the prefill call of one 8B projection (--m rows, default "
                         "2048 here; --steps calls) and print its TFLOP/s, nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(no collectives are part of the path)", file=sys.stderr)
        sys.exit(2)

    import torch
    import izwi_amd as qa

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    qa.lib()
    dtype = Q4_K if args.workload == "decode_q4k_8b_stack" else Q8_0

    if args.batched_percall:
        print(json.dumps({"batched_percall_us": batched_percall(torch, qa, dtype, args.m if args.m >= 3 else 16),
                          "m": args.m if args.m >= 3 else 16, "dtype": "Q4_K" if dtype == Q4_K else "Q8_0"}))
        return

    if args.neighbours_only:
        print(json.dumps({"decode_step_neighbours_f32": neighbours_extra(torch, qa, args.steps, args.warmup)}))
        return

    if args.moe_only:
        import numpy as np
        e, top_k, hidden, inter, t = 128, 8, 2048, 768, args.m
        gg = qa.GgmlDType(Q4_K)

        def stack(n, k, seed):
            return qa.QTensor.from_blocks(gg, np.tile(make_blocks(Q4_K, 8 * n, k, seed), e // 8), (e, n, k))
        experts = qa.MoeExperts(stack(inter, hidden, 31), stack(inter, hidden, 32), stack(hidden, inter, 33))
        x = torch.from_numpy(synth_normal(40 + t, (t, hidden))).cuda()
        logits = torch.from_numpy(synth_normal(50 + t, (t, e))).cuda()
        ms = time_eager(torch, lambda: experts.layer(logits, x, top_k), args.steps, args.warmup)
        print(json.dumps({"moe_layer_us": round(ms * 1e3, 1), "tokens": t, "experts": e, "top_k": top_k}))
        return

    if args.prefill_only:
        m = args.m if args.m > 1 else 2048
        tf = prefill_extra(torch, qa, dtype, m, args.steps, args.warmup, only=args.prefill_only, form=args.prefill_form)
        print(json.dumps({"prefill_only": args.prefill_only, "m": m, "dtype": "Q4_K" if dtype == Q4_K else "Q8_0",
                          "form": args.prefill_form or "default", "tflops": tf[args.prefill_only]}))
        return

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # 1 GiB read + 1 GiB written by one elementwise copy kernel
        torch.cuda.synchronize()
        del src, dst

    weights = build_decode_weights(torch, qa, dtype, args.layers, True)
    make_calls = grouped_decode_calls if args.calls == "grouped" else decode_calls
    calls, total_bytes = make_calls(torch, dtype, weights, args.m)
    launches = len(calls)
    ms, _graph = time_graph(torch, lambda: run_calls(qa, calls), args.steps, args.warmup)
    gbs = total_bytes / (ms * 1e-3) / 1e9
    eager_ms = time_eager(torch, lambda: run_calls(qa, calls), max(3, args.steps // 5), 2)

    result = {
        "metric": "quant GEMV HBM GB/s (% peak) + prefill GEMM TFLOPS, Qwen3 shapes, 1 MI355X",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8 block dots, f32 scale/accumulate" if args.m <= 64 else "bf16",
        "data": "synthetic: seeded N(0,0.02) weights quantized to "
                f"{'Q4_K' if dtype == Q4_K else 'Q8_0'}, N(0,1) f32 activations; every layer has its own "
                "device buffers (same seeded bytes per projection kind); lm_head repeats 16384 seeded rows",
        "config": {
            "workload": f"{args.workload}: Qwen3-8B shapes, {args.layers} layers x 7 projections + lm_head, "
                        f"M={args.m}, {launches} calls/step ("
                        + ("qkv and gate/up as one projection-group call each, o / down / lm_head single calls: "
                           "the calls of the reference's Qwen3Attention::forward and Qwen3Mlp::forward"
                           if args.calls == "grouped" else "one call per projection")
                        + f"), {total_bytes / 1e9:.3f} GB algorithmic bytes/step, HIP-graph replay",
            "m": args.m,
            "calls": args.calls,
            "launches_per_step": launches,
            "algorithmic_bytes_per_step": int(total_bytes),
        },
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "eager_ms_per_step": round(eager_ms, 4),
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_kernel (fused activation-quantize + block-dot decode kernel)",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic(f"{args.workload}:{args.calls}", args.m, total_bytes / launches),
            "avg_launch_us": round(ms * 1e3 / launches, 3),
            "avg_algorithmic_bytes_per_launch": int(total_bytes / launches),
            "floor": None,  # filled below from the read-only launches of the same structure (extras)
        },
    }
    del calls, _graph

    extras = {}
    if not args.no_extras:
        # the same stack at the other decode batch sizes of the configuration
        try:
            for m in (8, 16):
                if m == args.m:
                    continue
                c, tb = make_calls(torch, dtype, weights, m)
                t, g = time_graph(torch, lambda: run_calls(qa, c), max(5, args.steps // 5), 3)
                extras[f"decode_gbs_m{m}"] = round(tb / (t * 1e-3) / 1e9, 1)
                extras[f"decode_ms_per_step_m{m}"] = round(t, 4)
                del c, g
            if args.calls == "grouped":
                for m in (8, 16):
                    extras[f"decode_records_path_m{m}"] = records_path_extra(torch, qa, dtype, weights, m)
            # the other call structure at the headline's m
            other = decode_calls if args.calls == "grouped" else grouped_decode_calls
            c, tb = other(torch, dtype, weights, args.m)
            t, g = time_graph(torch, lambda: run_calls(qa, c), max(5, args.steps // 2), 3)
            extras["decode_per_projection_calls" if args.calls == "grouped" else "decode_grouped_calls"] = {
                "gbs": round(tb / (t * 1e-3) / 1e9, 1), "ms_per_step": round(t, 4), "calls_per_step": len(c)}
            del c, g
            c, tb = make_calls(torch, dtype, weights, args.m)
            extras["decode_overlap_what_if"] = overlap_what_if_extra(torch, qa, c, tb)
            if args.m == 1 and args.calls == "grouped":
                extras["decode_chained_one_launch"] = chained_extra(torch, qa, c, tb)
            del c
            extras["decode_host_pointer_calls"] = host_pointer_extra(qa, weights, args.m)
            extras["hbm_ceiling_measured"] = hbm_ceiling_extra(torch)
            if args.calls == "grouped":
                floor = read_only_floor_extra(torch, qa, dtype, weights, args.m)
                extras["decode_read_only_floor"] = floor
                # what this launch structure allows: plain reads of the same bytes in the same dependent launches
                result["roofline"]["floor"] = {
                    "gbs": floor["gbs"], "frac_of_peak": round(floor["gbs"] / HBM_PEAK_GBS, 4),
                    "achieved_over_floor": round(gbs / floor["gbs"], 4),
                    "what": f"read-only launches of the same sizes in the same dependent chain of {launches} launches "
                            "(bench_probe_stream_read, 16-byte non-temporal loads, best launch shape per size): the "
                            "rate that one launch per projection call can reach on this GPU at these sizes"}
        except Exception as exc:  # extras never invalidate the headline number
            extras["decode_error"] = repr(exc)
    del weights
    torch.cuda.empty_cache()

    if not args.no_extras:
        try:
            pw = build_packed_weights(torch, qa, dtype, args.layers)
            c, tb = decode_calls(torch, dtype, pw, args.m)
            t, g = time_graph(torch, lambda: run_calls(qa, c), max(5, args.steps // 2), 3)
            extras["decode_packed_qkv_gateup"] = {
                "gbs": round(tb / (t * 1e-3) / 1e9, 1), "ms_per_step": round(t, 4), "launches_per_step": len(c),
                "note": "same projections, q|k|v and gate|up as one packed weight each (the reference's "
                        "packed_qmatmul_from_qtensors); not the headline: the reference packs on Metal only"}
            del pw, c, g
            torch.cuda.empty_cache()
        except Exception as exc:
            extras["decode_packed_error"] = repr(exc)
        try:
            # the other block format of the configuration on the same stack and call structure
            other_dtype = Q8_0 if dtype == Q4_K else Q4_K
            ow = build_decode_weights(torch, qa, other_dtype, args.layers, True)
            c, tb = make_calls(torch, other_dtype, ow, args.m)
            t, g = time_graph(torch, lambda: run_calls(qa, c), max(5, args.steps // 2), 3)
            extras["decode_q8_0_8b_stack" if other_dtype == Q8_0 else "decode_q4k_8b_stack"] = {
                "gbs": round(tb / (t * 1e-3) / 1e9, 1), "ms_per_step": round(t, 4),
                "pct_of_hbm_peak": round(100.0 * tb / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 2), "m": args.m,
                "calls_per_step": len(c)}
            del c, g
            other_key = "decode_q8_0_8b_stack" if other_dtype == Q8_0 else "decode_q4k_8b_stack"
            for m in (8, 16):  # the same stack at the other batch sizes of the configuration
                c, tb = make_calls(torch, other_dtype, ow, m)
                t, g = time_graph(torch, lambda: run_calls(qa, c), max(5, args.steps // 5), 3)
                extras[other_key][f"m{m}"] = {"gbs": round(tb / (t * 1e-3) / 1e9, 1), "ms_per_step": round(t, 4)}
                del c, g
            if args.calls == "grouped":
                floor = read_only_floor_extra(torch, qa, other_dtype, ow, args.m)
                extras["decode_q8_0_8b_stack" if other_dtype == Q8_0 else "decode_q4k_8b_stack"]["read_only_floor"] = {
                    "gbs": floor["gbs"], "ms_per_step": floor["ms_per_step"]}
            del ow
            torch.cuda.empty_cache()
        except Exception as exc:
            extras["decode_other_dtype_error"] = repr(exc)
        try:
            extras["small_configs_q8_0"] = small_configs_extra(torch, qa)
        except Exception as exc:
            extras["small_configs_error"] = repr(exc)
        try:
            extras["moe_30b_a3b_q4k"] = moe_extra(torch, qa)
        except Exception as exc:
            extras["moe_error"] = repr(exc)
        try:
            extras["decode_step_neighbours_f32"] = neighbours_extra(torch, qa)
        except Exception as exc:
            extras["neighbours_error"] = repr(exc)
        try:
            extras["decode_q4_k_m_mix_8b_stack"] = q4_k_m_mix_extra(torch, qa, 1)
            extras["decode_q4_k_m_mix_8b_stack_m16"] = q4_k_m_mix_extra(torch, qa, 16)
        except Exception as exc:
            extras["q4_k_m_mix_error"] = repr(exc)
        try:
            extras["qwen3_8b_decode_step_all_calls"] = layer_stack_extra(torch, qa, dtype)
        except Exception as exc:
            extras["layer_stack_error"] = repr(exc)
        try:
            extras["fused_call_and_q6k"] = fused_and_q6k_extra(torch, qa)
        except Exception as exc:
            extras["fused_q6k_error"] = repr(exc)
        try:
            extras["prefill_tflops_m2048_q4k"] = prefill_extra(torch, qa, Q4_K, 2048)
            extras["prefill_tflops_m2048_q8_0"] = prefill_extra(torch, qa, Q8_0, 2048)
            extras["prefill_tflops_m512_q4k"] = prefill_extra(torch, qa, Q4_K, 512)
            best = max(extras["prefill_tflops_m2048_q4k"].values())
            extras["prefill_best_frac_of_bf16_peak"] = round(best / BF16_PEAK_TFLOPS, 4)
            extras["prefill_tflops_m2048_q4k_plane_form"] = prefill_extra(torch, qa, Q4_K, 2048, form="plane")
            extras["prefill_library_bf16_gemm_m2048"] = library_gemm_extra(torch, 2048)
        except Exception as exc:  # extras never invalidate the headline number
            extras["error"] = repr(exc)
    if extras:
        result["extras"] = extras

    if not args.no_cpu_baseline:
        from oracle import oracle  # the checker, timed here as the CPU baseline; no other leg touches it
        result["cpu_baseline"] = cpu_baseline(oracle, dtype, args.m)
        if not args.no_extras:
            try:
                result["cpu_baseline"]["per_config"] = cpu_baseline_table(oracle, torch, qa)
            except Exception as exc:
                result["cpu_baseline"]["per_config_error"] = repr(exc)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
