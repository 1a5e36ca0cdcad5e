"""Several host threads calling the library at once on shared weight handles (pytest -m gpu).

The reference runs requests on parallel worker threads against one model
(crates/izwi-core/src/engine/executor/dispatch.rs:150-204, backends/policy.rs:28-30), so
`forward` must be callable concurrently on a shared weight.  The calls below all use the
library's per-stream scratch buffer (quantized activations, split-k partial tiles, the expert
MLP's intermediates): every thread's results must equal, bit for bit, what the same calls
give when one thread runs them alone."""
import sys
import threading

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = 8, 12
N_THREADS = 4
ROUNDS = 12


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def qa():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the HIP path cannot run (there is no fallback)")
    import izwi_amd
    izwi_amd.lib()
    torch.cuda.set_device(0)
    return izwi_amd


@pytest.fixture(scope="module")
def model(qa, oracle):
    """Shared handles: a Q4_K and a Q8_0 projection and a small expert stack."""
    def weight(dtype, n, k, seed):
        blocks = oracle.quantize(dtype, oracle.randn(seed, (n, k), std=0.02))
        return qa.QMatMul.from_qtensor(qa.QTensor.from_blocks(qa.GgmlDType(dtype), blocks, (n, k)))

    def stack(e, n, k, seed):
        blocks = oracle.quantize(Q4_K, oracle.randn(seed, (e * n, k), std=0.02))
        return qa.QTensor.from_blocks(qa.GgmlDType(Q4_K), blocks, (e, n, k))

    experts = qa.MoeExperts(stack(16, 256, 512, 903), stack(16, 256, 512, 904), stack(16, 512, 256, 905))
    return {"q4": weight(Q4_K, 1024, 4096, 901), "q8": weight(Q8_0, 512, 1024, 902), "experts": experts}


def thread_inputs(oracle, tid):
    """Every thread has its own activations: a call that read another thread's scratch shows."""
    cuda = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    return {
        "x5": cuda(oracle.randn(1000 + tid, (5, 4096))),
        "x16": cuda(oracle.randn(1100 + tid, (16, 4096))),
        "x40_q8": cuda(oracle.randn(1200 + tid, (40, 1024))),
        "xb512": cuda(oracle.randn(1300 + tid, (512, 4096))).to(torch.bfloat16),  # [1024 x 4096]: split along k
        "moe_x16": cuda(oracle.randn(1400 + tid, (16, 512))), "moe_l16": cuda(oracle.randn(1500 + tid, (16, 16))),
        "moe_x64": cuda(oracle.randn(1600 + tid, (64, 512))), "moe_l64": cuda(oracle.randn(1700 + tid, (64, 16))),
    }


def one_round(model, inp, order):
    """The calls of one round, in a thread-specific order (scratch sizes alternate); returns the outputs."""
    calls = {
        "f32_m5": lambda: model["q4"].forward(inp["x5"]),
        "f32_m16": lambda: model["q4"].forward(inp["x16"]),
        "q8_m40": lambda: model["q8"].forward(inp["x40_q8"]),
        "bf16_splitk": lambda: model["q4"].forward_bf16_to_f32(inp["xb512"]),
        "moe_t16": lambda: model["experts"].layer(inp["moe_l16"], inp["moe_x16"], 4),   # 4-row segments
        "moe_t64": lambda: model["experts"].layer(inp["moe_l64"], inp["moe_x64"], 4),   # 16-row tiles
    }
    names = sorted(calls)
    names = names[order % len(names):] + names[:order % len(names)]
    return {name: calls[name]() for name in names}


def run_threads(model, inputs, streams):
    results = [None] * N_THREADS
    errors = []
    start = threading.Barrier(N_THREADS)

    def work(tid):
        try:
            torch.cuda.set_device(0)
            start.wait()
            outs = []
            if streams is None:
                for r in range(ROUNDS):
                    outs.append(one_round(model, inputs[tid], tid + r))
            else:
                with torch.cuda.stream(streams[tid]):
                    for r in range(ROUNDS):
                        outs.append(one_round(model, inputs[tid], tid + r))
                streams[tid].synchronize()
            results[tid] = outs
        except Exception as exc:  # noqa: BLE001
            errors.append((tid, repr(exc)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(N_THREADS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=240)
    assert not any(t.is_alive() for t in threads), "a calling thread did not finish"
    torch.cuda.synchronize()
    assert not errors, errors
    return results


@pytest.mark.parametrize("mode", ["null_stream", "stream_per_thread"])
def test_concurrent_callers_match_single_thread(qa, oracle, model, mode):
    inputs = [thread_inputs(oracle, t) for t in range(N_THREADS)]
    _say(f"threads {mode}: single-thread reference")
    want = [one_round(model, inputs[t], 0) for t in range(N_THREADS)]
    torch.cuda.synchronize()
    streams = None if mode == "null_stream" else [torch.cuda.Stream() for _ in range(N_THREADS)]
    _say(f"threads {mode}: {N_THREADS} threads x {ROUNDS} rounds")
    got = run_threads(model, inputs, streams)
    for tid in range(N_THREADS):
        for r, outs in enumerate(got[tid]):
            for name, y in outs.items():
                assert torch.equal(y, want[tid][name]), (mode, tid, r, name)


def test_scratch_growth_keeps_old_buffers_alive(qa, oracle, model):
    """A call that outgrows the stream's scratch must not free the buffer earlier launches (or a
    captured graph) still address: capture a batched call, grow the scratch with a larger eager call
    on the same stream, replay."""
    s = torch.cuda.Stream()
    x = torch.from_numpy(oracle.randn(1800, (16, 4096))).cuda()
    with torch.cuda.stream(s):
        want = model["q4"].forward(x)          # allocates this stream's scratch (not capturable)
        s.synchronize()
        y = torch.empty_like(want)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            y.copy_(model["q4"].forward(x))
        g.replay()
        s.synchronize()
        assert torch.equal(y, want)
        big = torch.from_numpy(oracle.randn(1801, (64, 4096))).cuda()
        for m in (40, 64):                      # larger records
            model["q4"].forward(big[:m].contiguous())
        xb = torch.from_numpy(oracle.randn(1802, (2048, 4096))).cuda()
        model["q4"].forward(xb)                 # bf16 copy + split-k tiles: far beyond the first buffer
        s.synchronize()
        for _ in range(3):
            y.zero_()
            g.replay()
            s.synchronize()
            assert torch.equal(y, want)


def test_growth_during_capture_is_an_error_not_a_fault(qa, oracle, model):
    s = torch.cuda.Stream()
    x = torch.from_numpy(oracle.randn(1810, (16, 4096))).cuda()
    from izwi_amd import capi
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        failed = False
        try:
            with torch.cuda.graph(g, stream=s):
                try:
                    model["q4"].forward(x)     # fresh stream: no scratch yet, cannot allocate here
                except capi.QmmError as exc:
                    failed = True
                    assert "captur" in str(exc).lower()
        except RuntimeError:
            pass                                # torch may refuse to finish an empty / failed capture
        assert failed
    torch.cuda.synchronize()
    # reserving first makes the same capture legal
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        capi.check(capi.lib().izwi_qmm_scratch_reserve(1 << 20, s2.cuda_stream))
        want = None
        y = torch.empty((16, 1024), dtype=torch.float32, device="cuda")
        g2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g2, stream=s2):
            y.copy_(model["q4"].forward(x))
        g2.replay()
        s2.synchronize()
    want = model["q4"].forward(x)
    torch.cuda.synchronize()
    assert torch.equal(y, want)
