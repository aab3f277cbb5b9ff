"""Zero-element inputs through the C ABI: nothing is launched on an empty grid.

Entry points that take a flat tensor return an empty result; entry points that carry a channel geometry
(elements per channel) or accumulate statistics reject a zero-sized tensor with an error message instead of
launching a kernel on it.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


@pytest.fixture(scope="module")
def empty():
    return torch.empty(0, device="cuda")


def test_flat_entry_points_return_empty_results(ops, empty):
    one = torch.ones(1, device="cuda")
    results = [
        ops.qdq_per_tensor(empty, -1, 1, 8),
        ops.fp16_round_trip(empty),
        ops.bf16_round_trip(empty),
        ops.fp8_fake_cast(empty, one),
        ops.quantize_per_tensor(empty, -1, 1, 8, False),
        ops.ste_bwd_per_tensor(empty, empty, -1, 1),
        *ops.qdq_codes_per_tensor(empty, -1, 1, 8),
    ]
    torch.cuda.synchronize()
    for r in results:
        assert r.numel() == 0 and r.device.type == "cuda"


def test_channel_geometry_without_elements_is_rejected(ops, empty):
    from aimet_amd._lib import MiqError
    one = torch.ones(1, device="cuda")
    mn, mx, delta, offset = ops.per_channel_params(-one, one, 255)
    calls = [
        lambda: ops.qdq_per_channel(empty, 1, 0, mn, mx, delta, offset),
        lambda: ops.ste_bwd_per_channel(empty, empty, 1, 0, mn, mx),
        lambda: ops.v2_qdq(empty, 1, 0, one, 0 * one, -128, 127),
        lambda: ops.v2_qdq_bwd(empty, empty, 1, 0, one, 0 * one, -128, 127),
        lambda: ops.v2_qdq_bwd_params(empty, empty, 1, 0, one, 0 * one, -128, 127),
        lambda: ops.minmax_per_channel(empty, 1, 0),
    ]
    for call in calls:
        with pytest.raises(MiqError):
            call()
    torch.cuda.synchronize()


@pytest.mark.parametrize("mode", ["QUANTIZATION_TF", "QUANTIZATION_TF_ENHANCED"])
def test_an_empty_batch_is_rejected_and_leaves_the_statistics_alone(ops, empty, mode):
    from aimet_amd import _lib
    data = torch.randn(4096, device="cuda")
    plain, disturbed = ops.Analyzer(getattr(_lib, mode)), ops.Analyzer(getattr(_lib, mode))
    plain.update_stats(data)
    with pytest.raises(_lib.MiqError):
        disturbed.update_stats(empty)
    disturbed.update_stats(data)
    with pytest.raises(_lib.MiqError):
        disturbed.update_stats(empty)
    (a, a_valid), (b, b_valid) = plain.compute_encoding(8), disturbed.compute_encoding(8)
    assert a_valid and b_valid
    assert (a.min, a.max, a.delta, a.offset) == (b.min, b.max, b.delta, b.offset)
