"""The entry point that allocates nothing (wgml_attention_noalloc) against wgml_attention: same
launches, partial results in the library's fixed scratch array instead of a workspace from
hipMalloc.  Two calls in a row, the second with a smaller input (the array keeps the first
call's contents), each compared with the allocating entry point bit for bit and with the
oracle within the attention tolerance; a shape beyond the array is refused.  The free device
memory reported by hipMemGetInfo must not move across the calls, and a call recorded under
stream capture must replay correctly."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu


def run_case(gpu, seq_len, n_heads, kv_mul, head_size, pos, seed):
    kv_dim = n_heads // kv_mul * head_size
    rng = np.random.default_rng(seed)
    q = rng.standard_normal(n_heads * head_size).astype(np.float32)
    kc = rng.standard_normal((seq_len, kv_dim)).astype(np.float32)
    vc = rng.standard_normal((seq_len, kv_dim)).astype(np.float32)
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, head_size, pos)
    op = W.BatchedMultiqueryAttention.from_device(gpu)
    gq, gk, gv = (W.GpuVector.init(gpu, a.reshape(-1)) for a in (q, kc, vc))
    out_ref = W.GpuVector.init(gpu, np.zeros(n_heads * head_size, np.float32))
    out_new = W.GpuVector.init(gpu, np.zeros(n_heads * head_size, np.float32))
    op.dispatch_multi(p, gq, gk, gv, out_ref)
    op.dispatch_noalloc(p, gq, gk, gv, out_new)
    a, b = out_ref.read(), out_new.read()
    want, _ = orc.attention(seq_len, kv_dim, kv_mul, n_heads, head_size, pos, q, kc, vc)
    assert np.array_equal(a, b), float(np.abs(a - b).max())
    assert np.abs(b - want).max() <= 1e-4 * max(1.0, float(np.abs(want).max()))


def hip_runtime():
    """The HIP runtime the library itself is linked against: the copy already mapped into this
    process (another copy of the runtime, loaded by name, would know nothing of its device)."""
    paths = []
    for line in open("/proc/self/maps"):
        path = line.split()[-1]
        if "libamdhip64" in path and path not in paths:
            paths.append(path)
    assert paths, "libwgml_hip.so is loaded, so its HIP runtime must be mapped"
    # the library links /opt/rocm's runtime; a second copy (PyTorch ships one) may be mapped too
    paths.sort(key=lambda p: "torch" in p)
    return C.CDLL(paths[0])


def free_device_bytes(hip):
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_noalloc_attention_two_calls_in_a_row(gpu):
    # first call: long context, grouped queries: many partial results per head in the scratch
    run_case(gpu, seq_len=4096, n_heads=32, kv_mul=4, head_size=128, pos=4000, seed=1)
    # second call, smaller in every way (fewer heads, positions and partials): must not be
    # disturbed by what the first call left in the array
    run_case(gpu, seq_len=1024, n_heads=12, kv_mul=1, head_size=64, pos=300, seed=2)
    # a single-workgroup plan (no partials at all) and an odd head size (general kernel)
    run_case(gpu, seq_len=256, n_heads=8, kv_mul=2, head_size=64, pos=17, seed=3)
    run_case(gpu, seq_len=512, n_heads=6, kv_mul=1, head_size=50, pos=400, seed=4)


def test_noalloc_attention_refuses_what_the_array_cannot_hold(gpu):
    # 2048 query heads of 256 on one KV head: 2048 heads x 2 workgroups x (256 + 2) floats
    # = 4.2 MB of partial results > the 2 MiB array
    seq_len, n_heads, head_size, pos = 64, 2048, 256, 40
    p = W.BatchedMultiqueryAttentionParams(seq_len, head_size, n_heads, n_heads, head_size, pos)
    op = W.BatchedMultiqueryAttention.from_device(gpu)
    gq = W.GpuVector.uninit(gpu, n_heads * head_size)
    gk = W.GpuVector.uninit(gpu, seq_len * head_size)
    out = W.GpuVector.uninit(gpu, n_heads * head_size)
    with pytest.raises(W.WgmlError, match="fixed scratch array"):
        op.dispatch_noalloc(p, gq, gk, gk, out)
    op.dispatch_multi(p, gq, gk, gk, out)  # the allocating entry point takes the same shape
    gpu.synchronize()


def test_noalloc_attention_leaves_free_memory_unchanged(gpu):
    # the allocating entry point grows its workspace for a shape it has not seen (free memory
    # drops); the entry point under test must not move it, also for a shape seen for the first time
    hip = hip_runtime()
    seq_len, n_heads, kv_mul, hs, pos = 2048, 16, 2, 128, 1500
    kv_dim = n_heads // kv_mul * hs
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    op = W.BatchedMultiqueryAttention.from_device(gpu)
    rng = np.random.default_rng(8)
    gq = W.GpuVector.init(gpu, rng.standard_normal(n_heads * hs).astype(np.float32))
    gk = W.GpuVector.init(gpu, rng.standard_normal(seq_len * kv_dim).astype(np.float32))
    gv = W.GpuVector.init(gpu, rng.standard_normal(seq_len * kv_dim).astype(np.float32))
    out = W.GpuVector.init(gpu, np.zeros(n_heads * hs, np.float32))
    gpu.synchronize()
    before = free_device_bytes(hip)
    for _ in range(3):
        op.dispatch_noalloc(p, gq, gk, gv, out)
    gpu.synchronize()
    assert free_device_bytes(hip) == before


def test_noalloc_attention_under_stream_capture(gpu):
    # the call only launches kernels, so it can be recorded into a HIP graph: three replays with
    # the program's own eager work and synchronisations between them, every one checked against
    # the eager result for the inputs it ran on
    hip = hip_runtime()
    seq_len, n_heads, kv_mul, hs, pos = 1024, 8, 2, 128, 900
    kv_dim = n_heads // kv_mul * hs
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    op = W.BatchedMultiqueryAttention.from_device(gpu)
    rng = np.random.default_rng(9)
    gq = W.GpuVector.init(gpu, rng.standard_normal(n_heads * hs).astype(np.float32))
    gk = W.GpuVector.init(gpu, rng.standard_normal(seq_len * kv_dim).astype(np.float32))
    gv = W.GpuVector.init(gpu, rng.standard_normal(seq_len * kv_dim).astype(np.float32))
    out = W.GpuVector.init(gpu, np.zeros(n_heads * hs, np.float32))
    eager = W.GpuVector.init(gpu, np.zeros(n_heads * hs, np.float32))
    op.dispatch_noalloc(p, gq, gk, gv, out)  # untimed first use of the kernels, outside capture
    gpu.synchronize()
    stream = C.c_void_p(gpu.stream())
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    thread_local = 1  # hipStreamCaptureModeThreadLocal
    assert hip.hipStreamBeginCapture(stream, thread_local) == 0
    try:
        op.dispatch_noalloc(p, gq, gk, gv, out)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, C.c_size_t(0)) == 0
    try:
        for rep in range(3):
            gq.write(rng.standard_normal(n_heads * hs).astype(np.float32))  # eager work in between
            out.write(np.zeros(n_heads * hs, np.float32))
            gpu.synchronize()
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            gpu.synchronize()
            op.dispatch_multi(p, gq, gk, gv, eager)
            assert np.array_equal(out.read(), eager.read()), rep
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
