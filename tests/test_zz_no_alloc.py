"""mi355_gemmlowp_run_noalloc (the entry point that allocates nothing: its workspace is a fixed array on the device)
against mi355_gemmlowp_run on the same handle and inputs, to the same bar: identical bytes. Two calls in a row, the
second with a smaller input, so that what the first call left in the shared workspace is still there."""
import numpy as np
import pytest

import oracle
from computelibrary_amd import capi
from gpu_util import announce, to_dev

pytestmark = pytest.mark.gpu


def _case(M, N, K, lda, a_dt, b_dt, b_off, seed, run_first=True):
    """one handle, one input: (A on the device, handle, result of the allocating entry point, oracle result); with
    run_first False the handle is prepared but has never run"""
    import torch
    rng = np.random.default_rng(seed)
    A = rng.integers(np.iinfo(a_dt).min, np.iinfo(a_dt).max + 1, size=(M, K)).astype(a_dt)
    B = rng.integers(np.iinfo(b_dt).min, np.iinfo(b_dt).max + 1, size=(K, N)).astype(b_dt)
    bias = rng.integers(-3000, 3000, size=N, dtype=np.int32)
    mult, shift = oracle.calculate_quantized_multipliers(1.0, [3e-4 * 128.0 / np.sqrt(K)], 1.0)
    lo, hi = (-128, 127) if a_dt == np.int8 else (0, 255)
    code = capi.S8 if a_dt == np.int8 else capi.U8
    g = capi.Gemm(M, N, K, code, capi.S8 if b_dt == np.int8 else capi.U8, code, capi.EPI_FIXEDPOINT, -7, b_off,
                  capi.requant(int(mult[0]), int(shift[0]), 5, lo, hi), lda=lda)
    Ah = np.zeros((M, lda), dtype=a_dt)
    Ah[:, :K] = A
    Ad = to_dev(Ah)
    keep = [to_dev(B), to_dev(bias)]
    g.prepare(keep[0], keep[1])
    want = oracle.gemmlowp_fixedpoint(A, B, bias, -7, b_off, mult, shift, 5, lo, hi, a_dt)
    if not run_first:
        torch.cuda.synchronize()
        return Ad, g, None, want, keep
    D_ref = torch.zeros((M, N), dtype=torch.int8 if a_dt == np.int8 else torch.uint8, device="cuda")
    g.run(Ad, D_ref)
    torch.cuda.synchronize()
    return Ad, g, D_ref.cpu().numpy(), want, keep


@pytest.mark.parametrize("lda_extra", [0, 3])  # rows 16-byte aligned (row sums only) / unaligned (row sums + copy of A)
def test_noalloc_matches_the_allocating_entry_point_twice_in_a_row(lda_extra):
    import torch
    assert capi.lib().mi355_gemmlowp_noalloc_workspace_bytes() == 8 << 20
    shapes = [(300, 200, 528), (70, 96, 272)]  # the second call is smaller than the first
    for rep, (M, N, K) in enumerate(shapes):
        announce("no-alloc", (M, N, K), "lda +", lda_extra, "call", rep)
        Ad, g, ref, want, keep = _case(M, N, K, K + lda_extra, np.uint8, np.uint8, 9, 500 + rep)
        np.testing.assert_array_equal(ref, want)
        D = torch.full((M, N), 77, dtype=torch.uint8, device="cuda")
        g.run_noalloc(Ad, D)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(D.cpu().numpy(), ref)
        # and once more on the same handle: the workspace still holds this call's own values
        D.fill_(0)
        g.run_noalloc(Ad, D)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(D.cpu().numpy(), ref)
        g.close()


def test_noalloc_skinny_and_signed_paths():
    import torch
    for (M, N, K, a_dt, b_dt, b_off) in [(8, 256, 512, np.int8, np.int8, 11), (33, 130, 192, np.int8, np.int8, -4),
                                          (16, 64, 128, np.int8, np.int8, 0)]:
        announce("no-alloc", (M, N, K), a_dt.__name__, "b_off", b_off)
        Ad, g, ref, want, keep = _case(M, N, K, K, a_dt, b_dt, b_off, 600 + M)
        np.testing.assert_array_equal(ref, want)
        D = torch.zeros((M, N), dtype=torch.int8, device="cuda")
        g.run_noalloc(Ad, D)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(D.cpu().numpy(), ref)
        g.close()


def test_noalloc_rejects_what_does_not_fit_and_host_memory():
    import torch
    # unaligned rows: the padded copy of A would need 5000 * 2048 bytes > 8 MiB
    M, N, K = 5000, 32, 2045
    g = capi.Gemm(M, N, K, capi.S8, capi.S8, capi.S32, capi.EPI_S32, 0, 3, lda=K)
    Bd = torch.zeros((K, N), dtype=torch.int8, device="cuda")
    g.prepare(Bd)
    Ad = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    Dd = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.Mi355Error, match="workspace"):
        g.run_noalloc(Ad, Dd)
    with pytest.raises(capi.Mi355Error, match="device memory"):
        g.run_noalloc(np.zeros((M, K), np.int8), Dd)
    g.run(Ad, Dd)  # the allocating entry point still takes it
    torch.cuda.synchronize()
    g.close()


@pytest.mark.parametrize("lda_extra", [0, 3])
def test_noalloc_on_a_handle_that_never_ran_allocates_nothing(lda_extra):
    """The first run of a handle through the entry point that allocates nothing (the allocating one has not sized any
    workspace for it), and the device's free memory before and after: unchanged."""
    import torch
    M, N, K = 260, 136, 400
    # (a first handle takes whatever the first use of these kernels costs the process - code objects, the one-time set-up
    # of the workspace - out of the measurement)
    Ad, g, _, want, keep = _case(M, N, K, K + lda_extra, np.uint8, np.uint8, 9, 700, run_first=False)
    D = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
    g.run_noalloc(Ad, D)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(D.cpu().numpy(), want)
    g.close()
    Ad, g, _, want, keep = _case(M, N, K, K + lda_extra, np.uint8, np.uint8, 9, 701, run_first=False)
    D.fill_(3)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    announce("no-alloc, cold handle", (M, N, K), "lda +", lda_extra)
    for _ in range(3):
        g.run_noalloc(Ad, D)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    np.testing.assert_array_equal(D.cpu().numpy(), want)
    g.close()


def test_noalloc_refuses_a_second_stream_while_the_first_is_busy():
    """One workspace per GPU: calls on one stream follow each other; a call on another stream while kernels of the first
    are still queued is refused, and accepted once they are done. A run that needs no workspace (no B offset, aligned
    rows) is never refused."""
    import torch
    M, N, K = 1024, 1024, 4000
    Ad, g, ref, want, keep = _case(M, N, K, K + 3, np.int8, np.int8, 4, 800)  # (rows not dword aligned: a padded copy of A)
    Ad0, g0, ref0, want0, keep0 = _case(64, 64, 256, 256, np.int8, np.int8, 0, 801)
    D = torch.zeros((M, N), dtype=torch.int8, device="cuda")
    D0 = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    announce("no-alloc, two streams")
    with torch.cuda.stream(s1):
        torch.cuda._sleep(100_000_000)  # tens of milliseconds of queued work in front of the first stream's call
    g.run_noalloc(Ad, D, stream=s1.cuda_stream)
    with pytest.raises(capi.Mi355Error, match="still in use"):
        g.run_noalloc(Ad, D, stream=s2.cuda_stream)
    g0.run_noalloc(Ad0, D0, stream=s2.cuda_stream)  # nothing of it lives in the workspace
    torch.cuda.synchronize()
    g.run_noalloc(Ad, D, stream=s2.cuda_stream)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(D.cpu().numpy(), ref)
    np.testing.assert_array_equal(D0.cpu().numpy(), ref0)
    g.close()
    g0.close()


def test_noalloc_captured_in_a_hip_graph_on_a_handle_that_never_ran():
    """What the entry point is for: a handle that has only been prepared is run for the first time inside a stream
    capture (rows that are not dword aligned: the padded copy of A and the row sums live in the fixed workspace), and
    every replay - with eager work and synchronisations in between - reproduces the oracle's bytes. (The per-GPU set-up of
    the workspace happened in an earlier call of this process, outside any capture.)"""
    import torch
    M, N, K = 300, 200, 528
    Ad0, g0, _, want0, keep0 = _case(64, 64, 272, 275, np.uint8, np.uint8, 9, 900, run_first=False)
    D0 = torch.zeros((64, 64), dtype=torch.uint8, device="cuda")
    g0.run_noalloc(Ad0, D0)  # the set-up call
    torch.cuda.synchronize()
    np.testing.assert_array_equal(D0.cpu().numpy(), want0)
    g0.close()
    Ad, g, _, want, keep = _case(M, N, K, K + 3, np.uint8, np.uint8, 9, 901, run_first=False)
    D = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    announce("no-alloc, graph capture of a cold handle", (M, N, K))
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        g.run_noalloc(Ad, D, stream=torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        D.fill_(77)  # eager work between replays
        torch.cuda.synchronize()
        announce("no-alloc, graph replay", rep)
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(D.cpu().numpy(), want)
    g.close()
