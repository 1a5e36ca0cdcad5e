#!/usr/bin/env python3
"""Per-item time stamps of the Q4_K expert kernels of one MoE layer (128 experts, top-8, hidden 2048,
expert intermediate 768: the benchmark's layer), from a library built with the time stamps compiled in:

    make -C izwi_amd/csrc -B EXTRA=-DQMM_EXPERT_TRACE
    python3 izwi_amd/csrc/expert_trace.py 512          # tokens
    make -C izwi_amd/csrc -B                           # back to the library proper

Prints, per launch (gate | up: four-unit panels, down: three-unit panels), how long items of each tile
count live, when their tiles had landed, and when the CUs finish."""
import collections
import ctypes
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import bench  # noqa: E402  (the benchmark's synthetic weights and inputs)
import izwi_amd as qa  # noqa: E402
from izwi_amd import capi  # noqa: E402


def main():
    t = int(sys.argv[1]) if len(sys.argv) > 1 else 512
    lib = capi.lib()
    if not hasattr(lib, "izwi_qmm_expert_trace_read"):
        sys.exit("the library was not built with -DQMM_EXPERT_TRACE")
    e, top_k, hidden, inter = 128, 8, 2048, 768
    gg = qa.GgmlDType(bench.Q4_K)

    def stack(n, k, seed):
        return qa.QTensor.from_blocks(gg, np.tile(bench.make_blocks(bench.Q4_K, 8 * n, k, seed), e // 8), (e, n, k))
    experts = qa.MoeExperts(stack(inter, hidden, 31), stack(inter, hidden, 32), stack(hidden, inter, 33))
    x = torch.from_numpy(bench.synth_normal(40 + t, (t, hidden))).cuda()
    logits = torch.from_numpy(bench.synth_normal(50 + t, (t, e))).cuda()
    for _ in range(5):
        experts.layer(logits, x, top_k)
    torch.cuda.synchronize()
    buf = np.zeros(8 * 8192, dtype=np.uint64)
    rc = lib.izwi_qmm_expert_trace_read(ctypes.c_void_p(buf.ctypes.data), ctypes.c_size_t(buf.nbytes))
    if rc:
        sys.exit(f"izwi_qmm_expert_trace_read: {rc}")
    rec = buf.reshape(1024, 8, 8)
    for kind, name in ((0, "gate | up (four-unit panels)"), (1, "down (three-unit panels)")):
        items = []
        for i in range(512):
            w = rec[kind * 512 + i]
            w = w[w[:, 2] != 0]
            if len(w) == 0:
                continue
            items.append((w[:, 0].min(), w[:, 1].max(), w[:, 2].max(), int(w[0, 3]), int(w[0, 4]) & 15, int(w[0, 5]), i // 256))
        if not items:
            continue
        a = np.array(items, dtype=np.int64)
        t0 = a[:, 0].min()
        start, window, end = ((a[:, c] - t0) / 100.0 for c in range(3))
        print(f"{name}: {len(a)} items, {end.max():.1f} us from the first item's start to the last item's end")
        for tiles in sorted(set(a[:, 5])):
            for rnd in (0, 1):
                m = (a[:, 5] == tiles) & (a[:, 6] == rnd)
                if m.any():
                    print(f"  {tiles} tiles, {'first' if rnd == 0 else 'second'} item of its workgroup: {m.sum():4d} items, "
                          f"live {(end - start)[m].mean():5.1f} us ({(end - start)[m].min():.1f} - {(end - start)[m].max():.1f}), "
                          f"tiles landed after {(window - start)[m].mean():4.1f} us")
        cus = collections.defaultdict(list)
        for row, en in zip(a, end):
            hw = int(row[3])
            cus[(int(row[4]), (hw >> 8) & 15, (hw >> 12) & 1, (hw >> 13) & 7)].append(en)
        done = sorted(max(v) for v in cus.values())
        print(f"  {len(cus)} CUs; they finish {done[0]:.1f} / {done[len(done) // 2]:.1f} / {done[-1]:.1f} us (first / median / last)")


if __name__ == "__main__":
    main()
