"""The W4A16 GEMM entry point that allocates nothing (kmi_gemm_w4a16_noalloc): its split-K partial sums live in a
device array inside the library instead of a caller-owned workspace.  Checked through the C ABI against
kmi_gemm_w4a16 with a workspace, bit for bit (same kernels, same split), on two calls in a row, the second smaller;
plus the size limit."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
from oracle import kairos_oracle as O

pytestmark = pytest.mark.gpu


def test_no_alloc_entry_point_matches_workspace_entry_point():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from kairos_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    splits_seen = []
    for (M, N, K, seed) in [(96, 1024, 4096, 1), (32, 512, 2048, 2), (8, 4096, 4096, 3), (128, 4096, 4096, 4)]:
        print(f"no-alloc case M={M} N={N} K={K}", flush=True)
        p = O.prepare_weights(O.synth_weights(N, K, seed=seed))
        qw = torch.from_numpy(p["qweight"]).cuda()
        sc, sz = torch.from_numpy(p["scales"]).cuda(), torch.from_numpy(p["scaled_zeros"]).cuda()
        x_h = O.synth_acts(M, K, seed=seed + 10)
        x = torch.from_numpy(x_h).cuda()
        bias = torch.from_numpy(np.random.default_rng(seed).standard_normal(N).astype(np.float16)).cuda()
        want = torch.empty((M, N), dtype=torch.float16, device="cuda")
        _lib.check(lib.kmi_gemm_w4a16(want.data_ptr(), x.data_ptr(), qw.data_ptr(), sc.data_ptr(), sz.data_ptr(),
                                      bias.data_ptr(), M, N, K, 128, ws.data_ptr(), ws.numel(), st))
        got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        before = torch.cuda.memory_allocated()
        _lib.check(lib.kmi_gemm_w4a16_noalloc(got.data_ptr(), x.data_ptr(), qw.data_ptr(), sc.data_ptr(), sz.data_ptr(),
                                              bias.data_ptr(), M, N, K, 128, st))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K)
        ref = O.gemm_w4a16(x_h, p["qweight"], p["scales"], p["scaled_zeros"]).astype(np.float32) + bias.cpu().numpy().astype(np.float32)
        assert O.max_abs_rel(got.cpu().numpy(), ref.astype(np.float16)) < 1e-2
        splits_seen.append(lib.kmi_gemm_splits_for(0, M, N, K, 16 << 20))
    assert max(splits_seen) > 1, "no case exercised the built-in scratch"
    # beyond the maximum: refused, nothing launched
    rc = lib.kmi_gemm_w4a16_noalloc(got.data_ptr(), x.data_ptr(), qw.data_ptr(), sc.data_ptr(), sz.data_ptr(), None,
                                    1024, 4096, 4096, 128, st)
    assert rc == -4 and b"exceed" in lib.kmi_get_last_error_string()
