"""GPU tests of C-ABI entry points that are not kernel launches of the convolution itself."""

import pytest
import torch

from spio_amd.hip import driver

pytestmark = pytest.mark.gpu


def test_zero_fill_covers_exactly_the_requested_bytes():
    """Any alignment, any size: the bytes asked for are zero, their neighbours are untouched."""
    buf = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    for offset, size in ((0, 0), (0, 1), (3, 5), (1, 15), (15, 17), (16, 16), (7, 4099), (13, 600001), (0, 1 << 20)):
        buf.fill_(0xAB)
        driver.zero_fill_async(buf.data_ptr() + offset, size, stream)
        torch.cuda.synchronize()
        assert int(buf[offset : offset + size].max().item() if size else 0) == 0, (offset, size)
        assert bool((buf[:offset] == 0xAB).all()) and bool((buf[offset + size :] == 0xAB).all()), (offset, size)


def test_zero_fill_replays_from_a_hip_graph():
    """Recorded under stream capture (it is a kernel launch, not a memset node) and replayed
    three times with eager work and synchronisations between the replays."""
    buf = torch.empty(100003, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            driver.zero_fill_async(buf.data_ptr() + 5, 99990, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for trial in range(3):
        buf.fill_(trial + 1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(buf[5:99995].max().item()) == 0
        assert bool((buf[:5] == trial + 1).all()) and bool((buf[99995:] == trial + 1).all())
