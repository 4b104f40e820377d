"""The entry point that allocates nothing (smx_reduce_forces_device_noalloc) against the allocating one
(smx_reduce_forces_device), through the C ABI, on two calls in a row, the second on a smaller input."""
import ctypes as C

import numpy as np
import pytest

from tests import helpers as H


@pytest.mark.gpu
def test_no_alloc_reduction_matches_the_allocating_one(tmp_path):
    import torch
    from symmetrix_amd import _lib
    from symmetrix_amd.mace import MACE
    L = _lib.lib()
    model = H.tiny_model(K=16, L_max=1, n_pts=48, seed=23, zbl=True)
    path = H.write_model(model, tmp_path / "noalloc.json")
    eng = MACE(path, "float64")
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    for n_atoms, seed in ((90, 5), (40, 6)):            # the second call is smaller: stale scratch must not leak in
        pos, cell, sp = H.small_system(n_atoms, seed=seed)
        nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
        N, E = len(sp), len(ea["r"])
        t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dev, dtype=dt)
        d = [t(ea["node_types"], torch.int32), t(ea["num_neigh"], torch.int32), t(ea["neigh_indices"], torch.int32),
             t(ea["neigh_types"], torch.int32), t(ea["xyz"], torch.float64), t(ea["r"], torch.float64)]
        print(f"no-alloc reduction: {N} atoms, {E} edges", flush=True)
        eng.compute_device(N, *[x.data_ptr() for x in d], E, 0, 0, stream)
        F_ref, V_ref = eng.reduce_forces_device(N, d[2].data_ptr(), virial=True)
        # outputs start as garbage: every entry must be written
        F = torch.full((N, 3), 7.0, dtype=torch.float64, device=dev); V = torch.full((6,), 7.0, dtype=torch.float64, device=dev)
        rc = L.smx_reduce_forces_device_noalloc(eng._h, N, C.c_void_p(d[2].data_ptr()), C.c_void_p(F.data_ptr()),
                                                C.c_void_p(V.data_ptr()), C.c_void_p(stream))
        assert rc == 0, L.smx_last_error().decode()
        torch.cuda.synchronize()
        assert np.array_equal(F.cpu().numpy(), F_ref)          # same kernels, same order of sums: same bits
        assert np.array_equal(V.cpu().numpy(), V_ref)
        assert np.abs(F_ref).max() > 0 and np.abs(H.atom_forces(nl, eng.node_forces, N) - F_ref).max() <= 1e-8
        # more atoms than receivers: the extra atoms only send nothing and receive nothing
        F2 = torch.full((N + 3, 3), 7.0, dtype=torch.float64, device=dev)
        assert L.smx_reduce_forces_device_noalloc(eng._h, N + 3, C.c_void_p(d[2].data_ptr()), C.c_void_p(F2.data_ptr()),
                                                  None, C.c_void_p(stream)) == 0
        torch.cuda.synchronize()
        assert np.array_equal(F2.cpu().numpy()[:N], F_ref) and not F2.cpu().numpy()[N:].any()
    # an out-of-range sender cannot raise without a synchronisation: the outputs are NaN
    bad = d[2].clone(); bad[0] = N + 5
    assert L.smx_reduce_forces_device_noalloc(eng._h, N, C.c_void_p(bad.data_ptr()), C.c_void_p(F.data_ptr()),
                                              C.c_void_p(V.data_ptr()), C.c_void_p(stream)) == 0
    torch.cuda.synchronize()
    assert torch.isnan(F).all() and torch.isnan(V).all()
    # and a good call afterwards is clean again
    assert L.smx_reduce_forces_device_noalloc(eng._h, N, C.c_void_p(d[2].data_ptr()), C.c_void_p(F.data_ptr()),
                                              C.c_void_p(V.data_ptr()), C.c_void_p(stream)) == 0
    torch.cuda.synchronize()
    assert np.array_equal(F.cpu().numpy(), F_ref) and np.array_equal(V.cpu().numpy(), V_ref)
    # sizes beyond the fixed scratch array are refused before anything is launched
    rc = L.smx_reduce_forces_device_noalloc(eng._h, 262144 + 1, C.c_void_p(d[2].data_ptr()), C.c_void_p(F.data_ptr()), None,
                                            C.c_void_p(stream))
    assert rc == -1 and b"exceed the fixed scratch array" in L.smx_last_error()
