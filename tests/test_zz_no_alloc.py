"""The operator entry that allocates nothing (imexHipGemmBiasSiluBf16SplitKNoAlloc, include/imex_hip_ops.h)
against the entry that allocates its workspace, through the C ABI of libimex-hip-ops.so."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

def test_no_alloc_entry_matches_the_allocating_entry(host, orc, stream):
    ops = host.ops()
    assert ops.imexHipOpsFixedWorkspaceBytes() == host.kernels().imexHipStreamKWorkspaceBytes(256) == 4096 + (64 << 20)
    assert ops.imexHipOpsInit(stream.handle) == 0, ops.imexHipOpsLastError()
    assert ops.imexHipOpsInit(stream.handle) == 0  # a second call does nothing
    # two calls in a row on the one fixed workspace, the second on a smaller problem (fewer workgroups, so part
    # of the workspace keeps what the first call left there); every tile of both is split between workgroups
    for M, N, K in ((1024, 1280, 4096), (512, 768, 2048)):
        a = orc.fill_normal(M * K, "bf16", 61 + M, 0.0, 1.0).reshape(M, K)
        b = orc.fill_normal(K * N, "bf16", 62 + M, 0.0, 0.05).reshape(K, N)
        bias = orc.fill_normal(N, "f32", 63 + M, 0.0, 0.1)
        d_a, d_b, d_bias = stream.to_device(a), stream.to_device(b), stream.to_device(bias)
        outs = []
        for entry in (ops.imexHipGemmBiasSiluBf16SplitK, ops.imexHipGemmBiasSiluBf16SplitKNoAlloc):
            d_o = stream.to_device(np.full((M, N), 0x7FC1, np.uint16))
            rc = entry(stream.handle, int(d_a), int(d_b), int(d_bias), int(d_o), M, N, K)
            assert rc == 0, ops.imexHipOpsLastError()
            stream.wait()
            outs.append(stream.from_device(d_o, (M, N), np.uint16))
            stream.free(d_o)
        for p in (d_a, d_b, d_bias):
            stream.free(p)
        # the same kernel, grid and order of additions: the same bits
        assert np.array_equal(outs[0], outs[1]), (M, N, K)
        # ... and the right ones: the one-workgroup-per-tile kernel's, to a step of the output type
        plain = orc.bfloat_to_float(host.gemm_bias_silu(stream, a, b, bias))
        got = orc.bfloat_to_float(outs[1])
        assert np.all(np.abs(got - plain) <= 2.0 ** -7 * np.abs(plain) + 1e-4), (M, N, K)


def test_no_alloc_entry_refuses_what_it_cannot_do(host, stream):
    ops = host.ops()
    null = C.c_void_p(0)
    assert ops.imexHipGemmBiasSiluBf16SplitKNoAlloc(null, null, null, null, null, 256, 256, 64) == -1  # no queue
    assert b"queue" in ops.imexHipOpsLastError()
    assert ops.imexHipGemmBiasSiluBf16SplitKNoAlloc(stream.handle, null, null, null, null, -1, 256, 64) == -1
    assert ops.imexHipGemmBiasSiluBf16SplitKNoAlloc(stream.handle, null, null, null, null, 0, 256, 64) == 0  # an empty C
