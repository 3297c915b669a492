"""The matrix-rate probe the benchmark reports beside the nominal MFMA peak:
it launches, returns its flop count and writes nothing.  (What rate it reaches
is the benchmark's business: a correctness suite does not assert clocks.)"""
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
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        assert paged_ops.mfma_probe(iters, sink) == flops
    b.record()
    torch.cuda.synchronize()
    assert a.elapsed_time(b) > 0.0
    assert torch.equal(sink.cpu(), torch.full((16,), 7.0))
