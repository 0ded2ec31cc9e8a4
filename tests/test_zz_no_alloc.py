"""The entry point that allocates nothing, sofie_hip_qgemm_s8_noalloc, against sofie_hip_qgemm_s8 through the C ABI:
bit-identical outputs on the shapes that use scratch memory (a long K cut into slices; a B [K,N] whose rows are not
16-byte aligned and is transposed first), two calls in a row with the second on a smaller input, and the clear error
for a shape beyond the fixed array. This file is collected last: the calls before it have used the context's own
scratch buffer, the ones here must not depend on it."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu


def _pair(ctx, L, transB, A, B, scale, bias, zpy, relu, out):
    """The same product through both entry points; returns the two outputs as numpy."""
    lib, h, p = ctx.lib, ctx.h, ctx.ptr
    dA, dB = ctx.dev(A), ctx.dev(B)
    dS, dBias = ctx.dev(scale), ctx.dev(bias)
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    dtype = {L.OUT_S8: torch.int8, L.OUT_S32: torch.int32, L.OUT_F32: torch.float32}[out]
    res = []
    for fn in (lib.sofie_hip_qgemm_s8, lib.sofie_hip_qgemm_s8_noalloc):
        y = ctx.empty((M, N), dtype)
        y.fill_(77)
        ctx.check(fn(h, int(transB), M, N, K, p(dA), K, p(dB), B.shape[1], p(dS), p(dBias), zpy,
                     L.ACT_RELU if relu else L.ACT_NONE, p(y), N, out))
        ctx.sync()
        res.append(y.cpu().numpy())
    return res


def test_noalloc_entry_point_matches_the_allocating_one():
    from sofie_amd import lib as L
    from sofie_amd import ops as o
    ctx = o.Context(0)
    r = np.random.default_rng(5)
    # (M, N, K, transB): the first of each pair is the larger one, so the second call finds the array
    # holding the first call's partial sums / transposed matrix
    cases = [
        (512, 512, 8192, True), (130, 250, 8320, True),          # K in slices, then fewer and ragged tiles
        (256, 256, 16384, True), (128, 128, 9000 // 16 * 16, True),
        (4096, 2052, 1024, False), (2100, 4100, 528, False),     # B [K,N], ldb % 16 != 0: transposed into the array
        (192, 320, 256, True),                                    # needs no scratch memory at all
    ]
    for M, N, K, tB in cases:
        print("[noalloc] M=%d N=%d K=%d transB=%d" % (M, N, K, tB), flush=True)
        A = r.integers(-127, 128, (M, K)).astype(np.int8)
        B = r.integers(-127, 128, (N, K) if tB else (K, N)).astype(np.int8)
        scale = (r.uniform(20, 60, N) / (73.3 * 73.3 * np.sqrt(K))).astype(np.float32)
        scale[1::7] *= -1
        bias = r.integers(-5000, 5000, N).astype(np.int32)
        for out, zpy, relu in ((L.OUT_S8, -3, True), (L.OUT_S32, 0, False)):
            a, b = _pair(ctx, L, tB, A, B, scale, bias, zpy, relu, out)
            assert np.array_equal(a, b), (M, N, K, tB, out)
        if M * N * K <= 1 << 29:
            assert np.array_equal(b, oracle.igemm_s8(A, B, transB=tB) + bias[None, :])
    ctx.close()


def test_noalloc_first_on_a_fresh_context_allocates_nothing():
    """On a context that has made no call yet (its own scratch buffer does not exist), the no-allocation entry point
    runs the shapes that need scratch memory with the device's free memory unchanged across the call, and its results
    equal the oracle's: the large B [K,N] cases on sampled rows, the K-slice case in full."""
    from sofie_amd import lib as L
    from sofie_amd import ops as o
    r = np.random.default_rng(9)
    for M, N, K, tB in ((4096, 2052, 1024, False), (2100, 4100, 528, False), (256, 256, 16384, True)):
        print("[noalloc fresh] M=%d N=%d K=%d transB=%d" % (M, N, K, tB), flush=True)
        ctx = o.Context(0)
        lib, h, p = ctx.lib, ctx.h, ctx.ptr
        A = r.integers(-127, 128, (M, K)).astype(np.int8)
        B = r.integers(-127, 128, (N, K) if tB else (K, N)).astype(np.int8)
        dA, dB = ctx.dev(A), ctx.dev(B)
        y = ctx.empty((M, N), torch.int32)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        ctx.check(lib.sofie_hip_qgemm_s8_noalloc(h, int(tB), M, N, K, p(dA), K, p(dB), B.shape[1], None, None, 0, L.ACT_NONE,
                                                 p(y), N, L.OUT_S32))
        ctx.sync()
        assert torch.cuda.mem_get_info()[0] == free0
        got = y.cpu().numpy()
        rows = np.arange(M) if M * N * K <= 1 << 30 else np.sort(r.choice(M, 48, replace=False))
        assert np.array_equal(got[rows], oracle.igemm_s8(A[rows], B, transB=tB))
        # the allocating entry point on the same context afterwards: the same bytes
        y2 = ctx.empty((M, N), torch.int32)
        ctx.check(lib.sofie_hip_qgemm_s8(h, int(tB), M, N, K, p(dA), K, p(dB), B.shape[1], None, None, 0, L.ACT_NONE, p(y2), N, L.OUT_S32))
        ctx.sync()
        assert np.array_equal(y2.cpu().numpy(), got)
        ctx.close()


def test_noalloc_calls_from_two_contexts_take_turns():
    """Two contexts (two streams) whose no-allocation calls both use the device's one scratch array, enqueued back to
    back without a wait in between: the library orders them on the device, so each result equals the one the same
    context computes alone."""
    from sofie_amd import lib as L
    from sofie_amd import ops as o
    r = np.random.default_rng(10)
    M, N, K = 256, 256, 16384                       # K cut into slices: partial sums in the array
    ctxs = [o.Context(0, stream=torch.cuda.Stream()) for _ in range(2)]
    ops_ = []
    for c in ctxs:
        A = r.integers(-127, 128, (M, K)).astype(np.int8)
        B = r.integers(-127, 128, (N, K)).astype(np.int8)
        ops_.append((c.dev(A), c.dev(B), c.empty((M, N), torch.int32), A, B))
    torch.cuda.synchronize()
    for rep in range(6):
        for c, (dA, dB, y, _, _) in zip(ctxs, ops_):
            c.check(c.lib.sofie_hip_qgemm_s8_noalloc(c.h, 1, M, N, K, c.ptr(dA), K, c.ptr(dB), K, None, None, 0, L.ACT_NONE,
                                                     c.ptr(y), N, L.OUT_S32))
    for c in ctxs:
        c.sync()
    for c, (dA, dB, y, A, B) in zip(ctxs, ops_):
        assert np.array_equal(y.cpu().numpy(), oracle.igemm_s8(A, B, transB=True))
        c.close()


def test_noalloc_entry_point_rejects_what_does_not_fit():
    """A transposed copy of 33.7 MB does not fit the 32 MiB array: EINVAL with a message, nothing launched, nothing allocated."""
    from sofie_amd import lib as L
    from sofie_amd import ops as o
    ctx = o.Context(0)
    lib, h, p = ctx.lib, ctx.h, ctx.ptr
    M, N, K = 3000, 8196, 4112                     # B [K,N] with ldb % 16 != 0 needs N*K = 33.7 MB > 32 MiB
    A = ctx.dev(np.zeros((M, K), np.int8))
    B = ctx.dev(np.zeros((K, N), np.int8))
    S = ctx.dev(np.ones(N, np.float32))
    y = ctx.empty((M, N), torch.int8)
    y.fill_(9)
    free0 = torch.cuda.mem_get_info()[0]
    rc = lib.sofie_hip_qgemm_s8_noalloc(h, 0, M, N, K, p(A), K, p(B), N, p(S), None, 0, 0, p(y), N, L.OUT_S8)
    assert rc == L.EINVAL
    msg = lib.sofie_hip_last_error(h).decode()
    assert "no-allocation" in msg and str(N * K) in msg
    ctx.sync()
    assert torch.cuda.mem_get_info()[0] == free0
    assert bool((y == 9).all())
    # the allocating entry point takes the same shape
    assert lib.sofie_hip_qgemm_s8(h, 0, M, N, K, p(A), K, p(B), N, p(S), None, 0, 0, p(y), N, L.OUT_S8) == 0
    ctx.sync()
    assert not bool(y.any())
    ctx.close()
