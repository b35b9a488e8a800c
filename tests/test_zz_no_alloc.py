"""The entry point that allocates nothing: dgpp_launch_mma_gemv_fp4_bf16_static (split-K partial sums in the
library's file-scope device array) against dgpp_launch_mma_gemv_fp4_bf16 with a caller's workspace, bit for bit, on
two calls in a row - the second with a smaller input, so that it meets the first call's leftovers in the array."""
import numpy as np
import pytest

from dgpp_amd import hostgen as hg, launch as L
from gpu_util import dev, dev_empty, fp4_matrix, host, sync

pytestmark = pytest.mark.gpu

STATIC_BYTES = 8 << 20


def _case(seed, group, m, n, k):
    w = hg.normal_f32(seed, (n, k), 0.02)
    if group == 16:
        payload, scales, ws2 = hg.encode_nvfp4(w)
        glob = dev(np.array([1.0 / np.float32(ws2)], np.float32))
    else:
        payload, scales = hg.encode_mxfp4(w)
        glob = None
    act = hg.normal_bf16(seed + 1, (m, k))
    p_d, s_d, a_d = dev(payload), dev(scales), dev(act)
    return (p_d, s_d, glob, a_d), fp4_matrix(p_d, s_d, glob, n, k, group), a_d


@pytest.mark.parametrize("group", [16, 32])
def test_static_workspace_entry_point_matches_the_workspace_form(gpu, group):
    import torch
    # both shapes leave the unsplit grid under-filled and have k >= 2048, so the K parts really run in separate blocks
    shapes = [(8, 2048, 4096), (3, 1024, 2048)]
    keep = []
    for i, (m, n, k) in enumerate(shapes):
        hold, wm, a_d = _case(0x5A7A71C + 16 * i + group, group, m, n, k)
        keep.append(hold)
        parts = 4 if k >= 4096 else 2
        ws = dev_empty(parts * m * n, np.float32)
        ws.fill_(float("nan"))
        want, got = dev_empty((m, n + 8), np.uint16), dev_empty((m, n + 8), np.uint16)
        want.zero_()
        got.zero_()
        L.launch_mma_gemv_fp4_bf16(a_d, k, wm, want, m, n, k, n + 8, None, ws, ws.numel() * 4)
        # a warm-up call first (the first call on a device looks the array's address up and loads the kernel's code
        # object), then the driver's own count of free device memory around the call: an allocation inside the library
        # would show there, whoever made it
        L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, got, m, n, k, n + 8, None)
        sync()
        got.zero_()
        sync()
        free_before = torch.cuda.mem_get_info()[0]
        L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, got, m, n, k, n + 8, None)
        sync()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
        w_h, g_h = host(want, np.uint16), host(got, np.uint16)
        assert not np.isnan(hg.bf16_to_f32(g_h[:, :n])).any()
        assert np.array_equal(g_h, w_h), f"call {i}: static workspace != caller's workspace"
        # and both equal the unsplit launch (no workspace at all)
        plain = dev_empty((m, n + 8), np.uint16)
        plain.zero_()
        L.launch_mma_gemv_fp4_bf16(a_d, k, wm, plain, m, n, k, n + 8, None, None, 0)
        sync()
        assert np.array_equal(host(plain, np.uint16), g_h)


def test_static_workspace_entry_point_refuses_what_does_not_fit(gpu):
    # a launch that WOULD run split (129 row tiles x 4 activation tiles < 1024) and whose partial sums do not fit:
    # 4 * 64 * 8256 floats = 8.06 MiB > 8 MiB
    m, n, k = 64, 8256, 5120
    assert 4 * m * n * 4 > STATIC_BYTES and ((n + 63) // 64) * ((m + 15) // 16) < 1024
    fake = 0x10000
    wm = L.Fp4Matrix(fake, fake, fake, n, k, 16, 0, None)
    with pytest.raises(L.InvalidArgument, match="static workspace"):
        L.launch_mma_gemv_fp4_bf16_static(fake, k, wm, fake, m, n, k, 0, None)
    L.launch_mma_gemv_fp4_bf16_static(fake, k, wm, fake, 0, n, k, 0, None)     # m <= 0 returns silently


def test_static_workspace_entry_point_runs_unsplit_launches_of_any_size(gpu):
    """A launch whose row tiles fill the chip by themselves runs unsplit and needs no workspace: it is not refused for
    parts * m * n floats beyond the static array (here 4 * 64 * 17408 floats = 17.8 MB), and gives the plain launch's bits."""
    m, n, k = 64, 17408, 4096
    assert 4 * m * n * 4 > STATIC_BYTES and ((n + 63) // 64) * ((m + 15) // 16) >= 1024
    hold, wm, a_d = _case(0x5A7A900, 32, m, n, k)
    got, plain = dev_empty((m, n), np.uint16), dev_empty((m, n), np.uint16)
    L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, got, m, n, k, 0, None)
    L.launch_mma_gemv_fp4_bf16(a_d, k, wm, plain, m, n, k, 0, None, None, 0)
    sync()
    assert np.array_equal(host(got, np.uint16), host(plain, np.uint16))


def test_static_workspace_is_bound_to_one_stream_until_released(gpu):
    import torch
    m, n, k = 8, 2048, 4096
    hold, wm, a_d = _case(0x5A7AA00, 32, m, n, k)
    out = dev_empty((m, n), np.uint16)
    L.static_scratch_release()
    side = torch.cuda.Stream()
    L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, out, m, n, k, 0, None)
    with pytest.raises(L.InvalidArgument, match="another stream"):
        L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, out, m, n, k, 0, side)
    sync()
    L.static_scratch_release()
    L.launch_mma_gemv_fp4_bf16_static(a_d, k, wm, out, m, n, k, 0, side)     # bound to the side stream now
    sync()
    L.static_scratch_release()
