"""The entry point that allocates nothing (ftk_stacked_lstm_noalloc_f32) against the entry point it is a variant of
(ftk_stacked_lstm_opts_f32 with fp32 products and a caller workspace): the same kernel on the same operands, so the
results have to be bit-identical.  Two calls in a row share the library's per-device scratch; the second is smaller,
so it meets what the first left behind."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(seed, L, T, B, H):
    rng = np.random.default_rng(seed)
    xs = torch.from_numpy(rng.standard_normal((T, B, H)).astype(np.float32)).cuda()
    WU = torch.from_numpy(rng.uniform(-1 / 16, 1 / 16, (L, 2 * H, 4 * H)).astype(np.float32)).cuda()
    bs = torch.from_numpy(rng.uniform(-1 / 16, 1 / 16, (L, 4 * H)).astype(np.float32)).cuda()
    return xs, WU, bs


def test_noalloc_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    import fractaltensor_amd._core as core
    from oracle import c_oracle
    from oracle import kaleido_oracle as ko
    H = 256
    for seed, (L, T, B, dil) in enumerate([(6, 40, 96, [1, 2, 4, 8, 16, 32]), (3, 7, 40, None)]):
        print(f'noalloc case L{L} T{T} B{B} dil {dil}', flush=True)
        xs, WU, bs = _inputs(40 + seed, L, T, B, H)
        ws = torch.empty(core.stacked_lstm_workspace_bytes(L, T, B, H), dtype=torch.uint8, device='cuda')
        h_ref, c_ref = core.stacked_lstm(xs, WU, bs, dilations=dil, workspace=ws, products='f32', check=True)
        hsss = torch.full((L, T, B, H), float('nan'), device='cuda')
        csss = torch.full((L, T, B, H), float('nan'), device='cuda')
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()['allocation.all.allocated']
        core.stacked_lstm_noalloc(xs, WU, bs, (hsss, csss), dilations=dil)
        assert torch.cuda.memory_stats()['allocation.all.allocated'] == before   # torch's allocator was not asked either
        core.stacked_lstm_check(None)
        assert torch.equal(hsss, h_ref) and torch.equal(csss, c_ref)
        # the library's own allocations do not pass through torch: the driver's count of free bytes must not move
        # over a second, warmed-up call either
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        core.stacked_lstm_noalloc(xs, WU, bs, (hsss, csss), dilations=dil)
        core.stacked_lstm_check(None)
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, (free_before, free_after)
        assert torch.equal(hsss, h_ref) and torch.equal(csss, c_ref)
        hr, cr = c_oracle.stacked_lstm(xs.cpu().numpy(), WU.cpu().numpy(), bs.cpu().numpy(), dil)
        assert ko.max_rel_err(hsss.cpu().numpy(), hr) <= 1e-4 and ko.max_rel_err(csss.cpu().numpy(), cr) <= 1e-4


def test_noalloc_entry_point_rejects_what_does_not_fit():
    import fractaltensor_amd._core as core
    xs, WU, bs = _inputs(1, 1, 2, 32, 128)                       # H != 256
    out = (torch.empty((1, 2, 32, 128), device='cuda'), torch.empty((1, 2, 32, 128), device='cuda'))
    with pytest.raises(core.FtkError) as info:
        core.stacked_lstm_noalloc(xs, WU, bs, out)
    assert info.value.code == -2
    # flags and trace beyond the 2 MiB scratch: L 32 x T 4096 x 8 row blocks of flags alone are 64 MiB.  Only the sizes
    # are looked at before the refusal, so small buffers stand in for the operands.
    import ctypes
    one = ctypes.c_void_p(xs.data_ptr())
    ci = ctypes.c_int
    rc = core.lib.ftk_stacked_lstm_noalloc_f32(one, one, None, None, one, one, ci(32), ci(4096), ci(256), ci(256), None)
    assert rc == -2 and b'scratch' in core.lib.ftk_last_error()
