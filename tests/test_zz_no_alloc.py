"""The entry point that allocates nothing: alpha_dconv3D_deltaW_GemmSK_static keeps its split-K partial sums in a static
device array of the library. Its result must equal, bit for bit, what alpha_dconv3D_deltaW_GemmSK + alpha_buf_summary give
with a caller-supplied deltaW_buf - also on a second call with a smaller layer, which finds the first call's partial sums
still in the array - and agree with the fp64 oracle to the bar of the other backward-filter tests."""
import numpy as np
import pytest

from oracle import oracle as O
from util import Dev, load_package, normal, out_dim

pkg = load_package()
DW = pkg.Cuda_dconv3D_deltaW

# N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ - the second and fourth are smaller than the ones before them
CALLS = [
    (8, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1, 16),
    (4, 9, 9, 16, 16, 3, 3, 1, 1, 1, 1, 5),
    (8, 28, 28, 128, 64, 1, 1, 1, 1, 0, 0, 8),
    (4, 13, 11, 36, 44, 3, 3, 2, 2, 1, 1, 3),
    (4, 8, 8, 32, 32, 3, 3, 1, 1, 1, 1, 1),
]


@pytest.mark.gpu
def test_static_scratch_entry_equals_the_workspace_entry_on_consecutive_calls():
    dev = Dev()
    torch = dev.torch
    for i, (N, IH, IW, IC, OC, FH, FW, sh, sw, ph, pw, GridZ) in enumerate(CALLS):
        OH, OW = out_dim(IH, IW, FH, FW, sh, sw, ph, pw)
        X, dY = normal((N, IH, IW, IC), 9100 + i), normal((N, OH, OW, OC), 9200 + i)
        x, dy = dev.put(X), dev.put(dY)
        sizeW = OC * FH * FW * IC
        print("static-scratch dW call %d: %s" % (i, CALLS[i]), flush=True)
        # the existing pair with a workspace from the caller
        ref = dev.guarded(OC, FH, FW, IC)
        buf = dev.empty(max(GridZ - 1, 1), sizeW, fill=float("nan"))
        DW.dconv3D_deltaW_GemmSK(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, ref.data_ptr(), buf.data_ptr(),
                                 FH, FW, N, IC, OC, sh, sw, ph, pw)
        DW.buf_summary(dev.stream, buf.data_ptr(), ref.data_ptr(), GridZ - 1, sizeW)
        want = dev.get(ref)
        # the entry under test. Device memory as the driver counts it (hipMemGetInfo: it sees an allocation made by any
        # library of the process, which the counters of PyTorch's caching allocator do not) must not move across the
        # call; the first call of the process resolves the static array's address and may load code, so it is made once
        # before the one that is measured.
        got_t = dev.guarded(OC, FH, FW, IC)
        if i == 0:
            DW.dconv3D_deltaW_GemmSK_static(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, got_t.data_ptr(),
                                            FH, FW, N, IC, OC, sh, sw, ph, pw)
            got_t.fill_(float("nan"))
        dev.sync()
        free_before = torch.cuda.mem_get_info()[0]
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        DW.dconv3D_deltaW_GemmSK_static(dev.streams, 1, GridZ, x.data_ptr(), IH, IW, dy.data_ptr(), OH, OW, got_t.data_ptr(),
                                        FH, FW, N, IC, OC, sh, sw, ph, pw)
        dev.sync()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory in use changed across the call"
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
        got = dev.get(got_t)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "call %d differs from GemmSK + buf_summary" % i
        oracle = O.deltaW_f64(X, dY, FH, FW, sh, sw, ph, pw)
        floor = 1e-5 * max(1.0, float(np.sqrt(np.mean(oracle * oracle))))
        assert O.max_err_ratio(got, oracle, 1e-4, floor) <= 1.0, "call %d vs oracle (rel 1e-4, abs %.2e)" % (i, floor)


def test_static_scratch_entry_refuses_what_does_not_fit():
    p = 256   # never dereferenced: the size check comes first, so this runs without a GPU
    # (GridZ - 1) * 512*3*3*512 floats = 9.4 MB * 4 per slice: GridZ 5 needs 37.7 MB > 32 MiB
    with pytest.raises(pkg.AlphaConvError, match="static scratch"):
        DW.dconv3D_deltaW_GemmSK_static([0], 1, 5, p, 7, 7, p, 7, 7, p, 3, 3, 4, 512, 512, 1, 1, 1, 1)
