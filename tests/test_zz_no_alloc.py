"""ptoamd_gemm_mx_static, the entry point that allocates nothing: its scale re-layout runs in the library's static device
array.  Checked through the C ABI against ptoamd_gemm_mx_ws (same kernels, caller workspace) bit for bit, on two calls in
a row, the second with a smaller input, so that what the first call left in the array cannot leak into the second."""
import numpy as np
import pytest
import torch

import __graft_entry__ as ge
from oracle import binding as ob

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def pa():
    mod = ge.load_package()
    mod.init(0)
    return mod


def _case(pa, seed, m, n, k, typ):
    r = np.random.default_rng(seed)
    packed = typ == pa.E2M1
    a = r.integers(0, 256, (m, k // 2 if packed else k)).astype(np.uint8)
    b = r.integers(0, 256, (n, k // 2 if packed else k)).astype(np.uint8)
    if not packed:
        a[(a & 0x7F) == 0x7F] = 0x12  # E4M3 NaN codes
        b[(b & 0x7F) == 0x7F] = 0x12
    sa = r.integers(119, 135, (m, k // 32)).astype(np.uint8)
    sb = r.integers(119, 135, (n, k // 32)).astype(np.uint8)
    t = lambda x: torch.from_numpy(x).to(DEV)
    sa_zz = pa.mx_scale_relayout(t(sa), pa.MX_A_ND, pa.MX_A_ZZ, m, k // 32)
    sb_nn = pa.mx_scale_relayout(t(sb), pa.MX_B_DN, pa.MX_B_NN, k // 32, n)
    return (a, b, sa, sb), (t(a), t(b), sa_zz, sb_nn)


def test_static_scratch_entry_matches_the_workspace_entry_twice_in_a_row(pa, oracle):
    shapes = [(512, 768, 2048, pa.E4M3), (96, 160, 256, pa.E2M1)]   # the second call is smaller (and another operand type)
    cases = [_case(pa, 5 + i, m, n, k, typ) for i, (m, n, k, typ) in enumerate(shapes)]
    want = []
    for (m, n, k, typ), (_, (a, b, sa, sb)) in zip(shapes, cases):
        ws = torch.empty(pa.gemm_mx_workspace_bytes(m, n, k, pa.MX_A_ZZ, pa.MX_B_NN), dtype=torch.uint8, device=DEV)
        want.append(pa.gemm_mx(a, b, sa, sb, m, n, k, typ, typ, pa.F32, sa_layout=pa.MX_A_ZZ, sb_layout=pa.MX_B_NN, workspace=ws))
        assert pa.last_kernel().startswith("tile"), pa.last_kernel()
    outs = [torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV) for (m, n, _, _) in shapes]
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info(DEV)[0]   # the driver's own count: sees a hipMalloc made behind torch's back
    for (m, n, k, typ), (_, (a, b, sa, sb)), out in zip(shapes, cases, outs):   # back to back on one stream
        pa.gemm_mx_static(a, b, sa, sb, m, n, k, typ, typ, out, sa_layout=pa.MX_A_ZZ, sb_layout=pa.MX_B_NN)
        assert pa.last_kernel().startswith("tile"), pa.last_kernel()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before   # nothing went through torch's allocator either
    assert torch.cuda.mem_get_info(DEV)[0] == free_before                        # and the device's free memory did not move
    for (m, n, k, typ), ((a, b, sa, sb), _), out, ref_ws in zip(shapes, cases, outs, want):
        got = out.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref_ws.cpu().numpy().view(np.uint32)), (m, n, k)
        otyp = ob.E4M3 if typ == pa.E4M3 else ob.E2M1
        ref = oracle.matmul_mx(a, b, sa, sb, m, k, n, otyp, otyp)
        err = np.abs(got - ref).max() / np.abs(ref).max()
        assert err <= 2e-2, (m, n, k, err)   # the bar of the block-scaled MFMA path against the oracle


def test_static_scratch_entry_limits(pa):
    tiny = torch.zeros(64, dtype=torch.uint8, device=DEV)
    out = torch.zeros((16, 16), dtype=torch.float32, device=DEV)
    # 16384 x 16384 x 8192 in ZZ / NN: 8 MiB of re-laid scales, twice the array: refused before anything is touched
    assert pa.gemm_mx_workspace_bytes(16384, 16384, 8192, pa.MX_A_ZZ, pa.MX_B_NN) > pa.STATIC_SCRATCH_BYTES
    with pytest.raises(pa.PtoAmdError, match="static scratch"):
        pa.gemm_mx_static(tiny, tiny, tiny, tiny, 16384, 16384, 8192, pa.E4M3, pa.E4M3, out, sa_layout=pa.MX_A_ZZ,
                          sb_layout=pa.MX_B_NN)
    # the natural layouts need no scratch at all: any size passes the limit check (and then runs as ptoamd_gemm_mx does)
    r = np.random.default_rng(3)
    m, n, k = 64, 64, 128
    a = torch.from_numpy(r.integers(0, 0x78, (m, k)).astype(np.uint8)).to(DEV)
    s = torch.full((m, k // 32), 127, dtype=torch.uint8, device=DEV)
    o1 = torch.empty((m, n), dtype=torch.float32, device=DEV)
    pa.gemm_mx_static(a, a, s, s, m, n, k, pa.E4M3, pa.E4M3, o1)
    o2 = pa.gemm_mx(a, a, s, s, m, n, k, pa.E4M3, pa.E4M3, pa.F32)
    assert torch.equal(o1, o2)
