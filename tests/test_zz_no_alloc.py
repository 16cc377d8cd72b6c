"""The entry point that allocates nothing (n2d2hip_sat_weight_forward_static: the reductions' scratch is a static array
in device memory) against the entry point it is a variant of (n2d2hip_sat_weight_forward, caller's workspace), through
the C ABI: bit-identical quantized weights and statistics on two calls in a row, the second on a smaller tensor, which
leaves the tail of the scratch holding the first call's partial results; then against the CPU oracle to the quantizer's
tolerance (1e-5, a handful of elements on rounding ties one level off)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
MODES = {"default": 1, "symrange": 3}


def test_static_scratch_entry_point_matches_the_workspace_one():
    import torch
    from n2d2_amd import capi, runtime
    from oracle import oracle as orc
    lib, sp = capi.lib, runtime.stream_ptr
    rng = np.random.default_rng(5)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
    f32 = dict(dtype=torch.float32, device="cuda")
    # two calls in a row per case: 1024 blocks of partial results, then 3 blocks
    for mode, apply_scaling, outputs_size in (("symrange", 0, 1), ("default", 1, 512), ("symrange", 1, 64)):
        for n in (512 * 512 * 3 * 3, 700):
            print("static scratch", mode, apply_scaling, n, flush=True)
            w = rng.normal(0, 0.05, size=n).astype(np.float32)
            dw = dev(w)
            want_q, want_stats = torch.empty(n, **f32), torch.empty(2, **f32)
            ws = torch.empty(int(lib.n2d2hip_quantizer_workspace_bytes(n)), dtype=torch.uint8, device="cuda")
            capi.check(lib.n2d2hip_sat_weight_forward(dw.data_ptr(), want_q.data_ptr(), n, 15.0, MODES[mode], apply_scaling, outputs_size,
                                                      want_stats.data_ptr(), ws.data_ptr(), ws.numel(), sp()))
            got_q, got_stats = torch.full((n,), -7.0, **f32), torch.full((2,), -7.0, **f32)
            capi.check(lib.n2d2hip_sat_weight_forward_static(dw.data_ptr(), got_q.data_ptr(), n, 15.0, MODES[mode], apply_scaling,
                                                             outputs_size, got_stats.data_ptr(), sp()))
            torch.cuda.synchronize()
            assert torch.equal(got_stats, want_stats), (mode, n)
            assert torch.equal(got_q, want_q), (mode, n)
            ref_q, tmax, scal = orc.sat_weight_forward(w.astype(np.float64) if apply_scaling else w, 15.0, mode,
                                                       apply_scaling=bool(apply_scaling), outputs_size=outputs_size)
            st = got_stats.cpu().numpy()
            assert abs(st[0] - tmax) <= 1e-5 * tmax and abs(st[1] - scal) <= 1e-5 * scal
            bad = np.abs(got_q.cpu().numpy().astype(np.float64) - ref_q) > 1e-5 * np.abs(ref_q).max()
            assert bad.sum() <= max(2, int(2e-4 * n)), (mode, n, int(bad.sum()))
    # beyond the stated maximum: a clear error, nothing launched
    rc = lib.n2d2hip_sat_weight_forward_static(dw.data_ptr(), got_q.data_ptr(), (1 << 28) + 1, 15.0, 3, 0, 1, got_stats.data_ptr(), sp())
    assert rc == capi.ERR_UNSUPPORTED and b"static scratch" in lib.n2d2hip_last_error()
    assert lib.n2d2hip_sat_weight_forward_static(None, got_q.data_ptr(), 8, 15.0, 3, 0, 1, got_stats.data_ptr(), sp()) == capi.ERR_INVALID
