"""The allocation-free forward of the fused lm_head + softcapped CE (ngpt_lmhead_ce_fwd_static, its workspace a
static device array inside the library) against the workspace-taking entry point, through the C ABI: two
calls in a row, the second on a smaller input, every output bit-equal; nothing is allocated by the call."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_PREDICT = 4


def _inputs(M, K, V, seed, n_predict, prefix):
    g = torch.Generator().manual_seed(seed)
    d = "cuda"
    x = torch.randn(M, K, generator=g).bfloat16().to(d)
    w = (torch.randn(V, K, generator=g) / math.sqrt(K)).bfloat16().to(d)
    t = torch.randint(0, V - 40, (M,), generator=g).to(d)
    mtp = torch.tensor([1.0, 0.5, 0.25, 0.125][:n_predict]).to(d)
    pt = (torch.randint(-1, V, (M,), generator=g) if prefix else torch.full((M,), -1)).to(d)
    pw = torch.tensor([0.3 if prefix else 0.0]).to(d)
    return x, w, t, mtp, pt, pw


def _outputs(M, K, V):
    d = "cuda"
    return dict(losses=torch.full((M,), float("nan"), device=d), lse=torch.full((M,), float("nan"), device=d),
                sig=torch.zeros((MAX_PREDICT + 1, M), device=d),
                x_f8=torch.zeros((M, K), dtype=torch.uint8, device=d), w_f8=torch.zeros((V, K), dtype=torch.uint8, device=d))


def test_static_forward_matches_the_workspace_forward_twice():
    import modded_nanogpt_amd as amd
    lib = amd._lib.load()
    assert torch.cuda.is_available()
    stream = torch.cuda.current_stream().cuda_stream
    x_s, w_s = 100 / 448, 1.6 / 448
    assert lib.ngpt_lmhead_ce_fwd_static_max_rows() == 65536
    # first a large call (many token tiles and all four vocabulary splits), then a smaller one with other options:
    # what the first call left in the library's buffer must not show in the second
    for (M, K, V, n_predict, prefix, layout) in [(4096, 256, 5120, 1, False, 0), (640, 128, 2432, 3, True, 0), (256, 128, 512, 1, False, 1)]:
        x, w, t, mtp, pt, pw = _inputs(M, K, V, seed=M + V, n_predict=n_predict, prefix=prefix)
        if layout == 1:
            w = w.T.contiguous()
        ref, got = _outputs(M, K, V), _outputs(M, K, V)
        # the built-in buffer holds the tables and partial sums only, i.e. the minimum workspace, which selects the tile
        # kernel: the reference call gets the same size, so both run the same kernel and every bit must agree
        nbytes = lib.ngpt_lmhead_ce_fwd_min_workspace_bytes(M, K, V, layout)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        common = (x.data_ptr(), w.data_ptr(), t.data_ptr(), mtp.data_ptr(), n_predict, pt.data_ptr(), pw.data_ptr(),
                  M, K, V, x_s, w_s, 23.0, 5.0, 7.5)
        outs = lambda o: (o["losses"].data_ptr(), o["lse"].data_ptr(), o["sig"].data_ptr(), o["x_f8"].data_ptr(), o["w_f8"].data_ptr())
        rc = lib.ngpt_lmhead_ce_fwd(*common, *outs(ref), layout, ws.data_ptr(), nbytes, stream)
        assert rc == 0, lib.ngpt_last_error()
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        torch_before = torch.cuda.memory_allocated()
        print(f"static forward M={M} K={K} V={V} n_predict={n_predict} prefix={prefix} layout={layout}", flush=True)
        rc = lib.ngpt_lmhead_ce_fwd_static(*common, *outs(got), layout, stream)
        assert rc == 0, lib.ngpt_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == torch_before
        assert torch.cuda.mem_get_info()[0] == free_before          # the device's free memory did not move either
        for name in ref:
            assert torch.isfinite(got[name].float()).all() or name in ("x_f8", "w_f8")
            assert torch.equal(got[name], ref[name]), name
    # beyond the built-in buffer: refused before anything is enqueued
    one = torch.zeros(1, device="cuda")
    rc = lib.ngpt_lmhead_ce_fwd_static(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), 1, None, None,
                                       65536 + 16, 128, 256, 1.0, 1.0, 23.0, 5.0, 7.5,
                                       one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), 0, stream)
    assert rc == -4 and b"65536" in lib.ngpt_last_error()
