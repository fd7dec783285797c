"""The allocation-free LayerNorm backward (``mi_layer_norm_bwd_static``: partial dW / dB slots in the
library's static device array) against the three-step path on caller-allocated partial buffers
(``mi_layer_norm_bwd_dx_partial_dwdb`` + ``mi_layer_norm_bwd_dwdb``, examples/layernorm.jl:245-251),
through the C ABI.

Bar: dX bit-exact (the same kernel computes it; it does not depend on the partial slots); dW / dB
within 1e-5 * (|ref| + max|ref|) of each other and of the float64 oracle (the slots are summed with
float atomics whose order differs from launch to launch).  Two calls in a row share the one static
array; the second is smaller, so stale contents of the first would show.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from cutile_jl_amd.examples import layernorm  # noqa: E402


def close_f32(got, ref, tol=1e-5):
    got = np.asarray(got, dtype=np.float64); ref = np.asarray(ref, dtype=np.float64)
    bound = tol * (np.abs(ref) + np.abs(ref).max())
    err = np.abs(got - ref)
    assert np.all(err <= bound), f"max err {err.max():.3e}, worst ratio {np.max(err / bound):.2f}"


def _both_paths(ct, orc, M, N, G, TILE_N):
    d = layernorm.prepare(M=M, N=N, GROUP_SIZE_M=G, seed=M + N)
    r = layernorm.run(d, TILE_N=TILE_N)           # forward + the three-step backward
    dx_ref, dw_ref, db_ref = r.DX.clone(), r.FINAL_DW.clone(), r.FINAL_DB.clone()
    d.DX.fill_(float("nan")); d.FINAL_DW.fill_(float("nan")); d.FINAL_DB.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    ct.layer_norm_bwd_static(d.DX, d.DY, d.X, d.W, d.Mean, d.Rstd, d.FINAL_DW, d.FINAL_DB, G, 32, TILE_N)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20), "the call took device memory"
    assert torch.equal(d.DX, dx_ref)
    close_f32(d.FINAL_DW.cpu().numpy(), dw_ref.cpu().numpy())
    close_f32(d.FINAL_DB.cpu().numpy(), db_ref.cpu().numpy())
    _, DW, DB = orc.layer_norm_bwd(orc.to_julia(d.X), orc.to_julia(d.W), orc.to_julia(d.DY), d.eps)
    close_f32(orc.to_julia(d.FINAL_DW), DW)
    close_f32(orc.to_julia(d.FINAL_DB), DB)


def test_static_backward_matches_three_step_path_twice(ct, orc):
    _both_paths(ct, orc, M=1024, N=4096, G=64, TILE_N=1024)   # first call: 64 slots of 4096
    _both_paths(ct, orc, M=130, N=1000, G=16, TILE_N=256)     # second, smaller: 16 slots of 1000
    _both_paths(ct, orc, M=7, N=30, G=4, TILE_N=32)           # rows that are no multiple of four


def test_static_backward_rejects_what_the_scratch_cannot_hold(ct):
    d = layernorm.prepare(M=4, N=16384, GROUP_SIZE_M=64)
    with pytest.raises(ct.MiError) as e:
        ct.layer_norm_bwd_static(d.DX, d.DY, d.X, d.W, d.Mean, d.Rstd, d.FINAL_DW, d.FINAL_DB, 64, 32, 1024)
    assert e.value.code == ct.MI_E_SCRATCH
