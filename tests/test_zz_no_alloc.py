"""cbk_gemm_static (the entry point that takes no workspace and allocates nothing) against cbk_gemm
on the same inputs, through the C ABI: the same kernels run in the same order, so the outputs are
bit-identical.  Two calls in a row, the second on a smaller input; a call recorded into a HIP graph
and replayed (after one eager call of the same configuration: the first call on a GPU looks up the
array's address, which cannot be recorded), with the allocator's counters unchanged across it; then
the refusal of a call that needs more scratch than the library's array holds."""
import ctypes

import pytest
import torch

from cobalt_amd import _lib, format as F, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _static(pm, x, out_dtype):
    M = x.shape[0]
    y = torch.full((M, pm.K), float("nan"), dtype=out_dtype, device=x.device)
    d = pm.desc()
    rc = _lib.lib().cbk_gemm_static(ctypes.byref(d), x.data_ptr(), F.dtype_code(x.dtype), M, x.stride(0), y.data_ptr(),
                                    F.dtype_code(out_dtype), pm.K, None, torch.cuda.current_stream().cuda_stream)
    return rc, y


def test_static_scratch_matches_cbk_gemm_twice():
    g = torch.Generator(device=DEV).manual_seed(3)
    big = F.synth_packed(768, 5376, F.BLK1632_4, seed=11, device=DEV).to_tiled()       # column range split: partial tiles too
    small = F.synth_packed(272, 1024, F.BLKC, 3, 64, 10, seed=12, device=DEV)
    for pm, M, dt in ((big, 300, torch.bfloat16), (small, 40, torch.float16)):          # the second call is the smaller one
        x = torch.randn(M, pm.N, device=DEV, generator=g).to(dt)
        want = ops.gemm(pm, x, out_dtype=torch.float32)
        rc, got = _static(pm, x, torch.float32)
        assert rc == 0, _lib.lib().cbk_strerror(rc).decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"M={M}: max diff {(got - want).abs().max().item()}"
    # and once more the larger one: the array still holds the smaller call's data
    x = torch.randn(300, big.N, device=DEV, generator=g).to(torch.bfloat16)
    rc, got = _static(big, x, torch.bfloat16)
    assert rc == 0
    assert torch.equal(got, ops.gemm(big, x))


def test_static_scratch_call_inside_a_graph_allocates_nothing():
    g = torch.Generator(device=DEV).manual_seed(5)
    pm = F.synth_packed(768, 5376, F.BLK1632_4, seed=13, device=DEV).to_tiled()
    M = 300
    x = torch.randn(M, pm.N, device=DEV, generator=g).to(torch.bfloat16)
    want = ops.gemm(pm, x, out_dtype=torch.float32)
    y = torch.full((M, pm.K), float("nan"), dtype=torch.float32, device=DEV)
    d = pm.desc()
    L = _lib.lib()

    def call(stream):
        return L.cbk_gemm_static(ctypes.byref(d), x.data_ptr(), F.dtype_code(x.dtype), M, x.stride(0), y.data_ptr(),
                                 F.F32, pm.K, None, stream)

    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        assert call(st.cuda_stream) == 0                       # eager: address lookup, kernel attributes
        st.synchronize()
        assert torch.equal(y, want)
        before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
        assert call(st.cuda_stream) == 0
        st.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=st):
            assert call(st.cuda_stream) == 0
        for _ in range(3):                                     # every replay against the eager result
            y.fill_(float("nan"))
            st.synchronize()
            graph.replay()
            st.synchronize()
            assert torch.equal(y, want)
    torch.cuda.current_stream().wait_stream(st)


def test_static_scratch_refuses_what_does_not_fit():
    pm = F.synth_packed(256, 21504, F.BLK1632_4, seed=1, device=DEV)
    M = 4096                                                                           # 4096 x 21504 fp16 = 168 MiB
    assert _lib.lib().cbk_workspace_bytes(ctypes.byref(pm.desc()), M) > (16 << 20)
    x = torch.zeros(M, pm.N, dtype=torch.bfloat16, device=DEV)
    rc, _ = _static(pm, x, torch.bfloat16)
    assert rc == -6                                                                    # CBK_ERR_WORKSPACE, nothing launched
