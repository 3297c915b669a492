"""The matrix-rate probe the benchmark reports beside the nominal MFMA peak:
it launches, returns its flop count, writes nothing, and times plausibly."""
import pytest
import torch

from ironcore_amd import paged_ops

pytestmark = pytest.mark.gpu


def test_probe_launches_and_counts_its_flops(gpu):
    sink = torch.full((16,), 7.0, dtype=torch.float32, device=gpu)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    iters = 2000
    flops = paged_ops.mfma_probe(iters, sink)
    assert flops == cus * 4 * iters * 16 * 2 * 32 * 32 * 16
    for _ in range(5):  # let the clock come up
        paged_ops.mfma_probe(iters, sink)
    best = 0.0
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        paged_ops.mfma_probe(iters, sink)
        b.record()
        torch.cuda.synchronize()
        best = max(best, flops / (a.elapsed_time(b) * 1e-3) / 1e12)
    assert torch.equal(sink.cpu(), torch.full((16,), 7.0))
    # a bare MFMA loop: above anything a real kernel reaches, never above the nominal peak
    assert 500.0 < best < 2600.0, best
