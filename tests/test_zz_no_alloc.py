"""The entry point that allocates nothing (gcmi_gemm_bf16_noalloc) against gcmi_gemm_bf16 on K-sliced shapes: the
same bits, on two calls in a row (the second smaller: the static scratch still holds the first call's partial
sums), in both weight layouts, and a clear error beyond the scratch's size."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _noalloc(gc, A, B, trans_b, bias, act, out):
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    return gc.lib().gcmi_gemm_bf16_noalloc(A.data_ptr(), B.data_ptr(), out.data_ptr(), M, N, K, K, B.shape[1], N, int(trans_b),
                                           None if bias is None else bias.data_ptr(), gc.BF16, gc.ACT[act], gc.BF16, s)


@pytest.mark.parametrize("trans_b", [False, True])
def test_noalloc_matches_the_allocating_entry_point_on_two_calls_in_a_row(gc, dev, trans_b):
    assert gc.lib().gcmi_noalloc_scratch_bytes() == 32 << 20
    shapes = [(64, 4096, 4096, "relu"), (32, 2048, 1024, None)]  # the second is smaller: stale partial sums stay behind it
    for M, N, K, act in shapes:
        assert gc.lib().gcmi_gemm_bf16_workspace_bytes(M, N, K, int(trans_b)) > 0  # K-sliced: the scratch is used
    for rep in range(2):
        for M, N, K, act in shapes:
            torch.manual_seed(M + N + K + rep)
            A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
            B = (torch.randn(K, N) * 0.05).to(torch.bfloat16).to(dev)
            if trans_b:
                B = B.t().contiguous()
            bias = torch.randn(N).to(torch.bfloat16).to(dev)
            want = gc.gemm_bf16_nt(A, B, bias, act) if trans_b else gc.gemm_bf16(A, B, bias, act)
            got = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
            assert _noalloc(gc, A, B, trans_b, bias, act, got) == 0, gc.lib().gcmi_last_error().decode()
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K, rep)
            ref = (A.float() @ (B.float().t() if trans_b else B.float())) + bias.float()
            if act == "relu":
                ref = torch.relu(ref)
            assert (got.float() - ref).abs().max().item() <= 0.02 * ref.abs().max().item() + 0.05


def test_noalloc_shapes_without_k_slices_need_no_scratch(gc, dev):
    M = N = K = 512
    torch.manual_seed(1)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    B = (torch.randn(K, N) * 0.5).to(torch.bfloat16).to(dev)
    got = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    assert _noalloc(gc, A, B, False, None, None, got) == 0
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), gc.gemm_bf16(A, B).view(torch.int16))


def test_noalloc_rejects_what_does_not_fit_the_static_scratch(gc, dev):
    M, N, K = 512, 4096, 16384  # 8 slices of 512 x 4096 f32 partial sums: 64 MB
    assert gc.lib().gcmi_gemm_bf16_workspace_bytes(M, N, K, 0) > 32 << 20
    A = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(K, N, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    st = _noalloc(gc, A, B, False, None, None, out)
    msg = gc.lib().gcmi_last_error().decode()
    assert st == 2 and "static" in msg and "bytes of scratch" in msg, (st, msg)
    torch.cuda.synchronize()
    assert gc.gemm_bf16(A, B).abs().max().item() == 0  # the allocating entry point takes the same call


def test_noalloc_allocates_nothing_and_can_be_captured(gc, dev):
    """The property the entry point is named for: device memory in use does not change over K-sliced calls (the
    allocating entry point would grow the library's workspace on a fresh shape), and a call recorded into a HIP graph
    replays to the eager result (several replays with eager work in between: the graph names the static array, whose
    address never changes).  The allocating entry point refuses a capturing stream with a message that names the
    alternatives."""
    M, N, K = 192, 8192, 4096     # K-sliced, 12 MiB of partial sums: beyond the library workspace's first size
    assert gc.lib().gcmi_gemm_bf16_workspace_bytes(M, N, K, 0) > 8 << 20
    torch.manual_seed(3)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    B = (torch.randn(K, N) * 0.05).to(torch.bfloat16).to(dev)
    got = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert _noalloc(gc, A, B, False, None, None, got) == 0, gc.lib().gcmi_last_error().decode()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    eager = got.clone()
    side = torch.cuda.Stream()
    out_g = torch.zeros_like(got)
    with torch.cuda.stream(side):
        assert _noalloc(gc, A, B, False, None, None, out_g) == 0  # once outside the graph on this stream
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        g.capture_begin()
        rc = _noalloc(gc, A, B, False, None, None, out_g)
        # the allocating entry point on the capturing stream: refused, nothing recorded
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc_alloc = gc.lib().gcmi_gemm_bf16(A.data_ptr(), B.data_ptr(), out_g.data_ptr(), M, N, K, K, N, N, None, gc.BF16, 0,
                                           gc.BF16, s)
        msg = gc.lib().gcmi_last_error().decode()
        g.capture_end()
    side.synchronize()
    assert rc == 0
    assert rc_alloc == 2 and "captured" in msg and "gcmi_gemm_bf16_ws" in msg, (rc_alloc, msg)
    for rep in range(3):
        out_g.zero_()
        # eager work of the program's own between the replays, through the same static scratch
        small = torch.empty(32, 2048, dtype=torch.bfloat16, device=dev)
        assert _noalloc(gc, A[:32, :1024].contiguous(), B[:1024, :2048].contiguous(), False, None, None, small) == 0
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.int16), eager.view(torch.int16)), rep
