"""The allocation-free min/max entry point (miq_minmax_per_channel_static_f32: partial results in an array inside the
library instead of a caller workspace) against miq_minmax_per_channel_f32 with a workspace, through the C ABI:
identical values, on consecutive calls that share the array, the later ones on smaller inputs."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(x, c, npc):
    from aimet_amd._lib import check, lib
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws = torch.empty(int(lib.miq_minmax_workspace_bytes(c, x.numel(), npc)) // 4 + 2, device="cuda")
    want = torch.full((2, c), 7.0, device="cuda")
    got = torch.full((2, c), -7.0, device="cuda")
    check(lib.miq_minmax_per_channel_f32(x.data_ptr(), c, x.numel(), npc, want.data_ptr(), ws.data_ptr(), stream))
    check(lib.miq_minmax_per_channel_static_f32(x.data_ptr(), c, x.numel(), npc, got.data_ptr(), stream))
    return got.cpu(), want.cpu()


def test_static_scratch_minmax_matches_the_workspace_entry_point():
    torch.manual_seed(5)
    # (outer, channels, elements per channel): large first, then smaller inputs that leave most of the array's
    # previous contents in place; several partial pairs per channel, one pair per channel, per-tensor
    for outer, c, npc in ((2, 96, 50000), (1, 33, 4100), (1, 1, 1 << 22), (3, 5, 40000), (1, 1, 1000), (1, 7, 3)):
        x = torch.randn(outer, c, npc, device="cuda") * 3
        x.view(-1)[::101] = float("nan")                     # ignored by both
        got, want = _both(x, c, npc)
        assert torch.equal(got, want), (outer, c, npc)
        ref = torch.nan_to_num(x, nan=float("inf")).amin(dim=(0, 2)).cpu()
        assert torch.equal(got[0], ref)


def test_static_scratch_minmax_refuses_what_does_not_fit():
    from aimet_amd._lib import MiqError, check, lib
    x = torch.zeros(16, device="cuda")
    out = torch.zeros(2, device="cuda")
    n = 1 << 30                                              # 65536 partial pairs: twice the array
    assert lib.miq_minmax_workspace_bytes(1, n, n) > 32768 * 8
    with pytest.raises(MiqError, match="too large"):
        check(lib.miq_minmax_per_channel_static_f32(x.data_ptr(), 1, n, n, out.data_ptr(), None))


def test_init_is_idempotent():
    """miq_init prepares the static scratch's device address ahead of the first use (for callers that capture)."""
    from aimet_amd._lib import check, lib
    for _ in range(2):
        check(lib.miq_init())
