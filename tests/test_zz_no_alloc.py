"""The entry point that allocates nothing: clg_group_sum_static keeps the partial sums of GroupSum in a buffer inside
the library image instead of a caller-provided scratch tensor.  Called through the C ABI and compared, bit for bit,
with clg_group_sum on the same input -- twice in a row, the second time on a smaller input (the buffer keeps the
first call's contents) -- and sizes beyond the buffer are rejected."""
import pytest
import torch

from convlogic_amd.hip import _lib
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _both(lib, x, k, tau):
    features, batch = x.shape
    dt = _lib.dtype_code(x)
    stream = _lib.stream_ptr(x)
    want = torch.full((batch, k), float("nan"), dtype=x.dtype, device=x.device)
    got = torch.full((batch, k), float("nan"), dtype=x.dtype, device=x.device)
    nbytes = lib.clg_group_sum_scratch_bytes(dt, features, batch, k)
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _lib.check(lib.clg_group_sum(dt, x.data_ptr(), want.data_ptr(), scratch.data_ptr(), features, batch, k, tau, stream))
    _lib.check(lib.clg_group_sum_static(dt, x.data_ptr(), got.data_ptr(), features, batch, k, tau, stream))
    return got, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_group_sum_static_matches_group_sum_on_two_calls_in_a_row(dtype):
    lib = _lib.load()
    assert lib.clg_group_sum_static_max_bytes() == 1 << 20
    torch.manual_seed(7)
    big = torch.rand(10240, 256, device=DEV, dtype=dtype)              # last layer of the k = 32 CIFAR net: 16 row slices
    small = torch.rand(640, 37, device=DEV, dtype=dtype)               # fewer rows, ragged batch, one slice
    for x, k, tau in ((big, 10, 6.5), (small, 10, 2.0), (big[:1280].contiguous(), 5, 1.0)):
        got, want = _both(lib, x, k, tau)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and torch.isfinite(got).all()
        ref = x.double().reshape(k, x.shape[0] // k, x.shape[1]).sum(1).t() / tau
        assert (got.double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()


def test_group_sum_static_rejects_what_does_not_fit():
    lib = _lib.load()
    x = torch.rand(640, 65536, device=DEV)                             # 1 slice * 10 classes * 65536 samples * 4 B = 2.5 MiB
    out = torch.empty(65536, 10, device=DEV)
    rc = lib.clg_group_sum_static(0, x.data_ptr(), out.data_ptr(), 640, 65536, 10, 1.0, _lib.stream_ptr(x))
    assert rc != 0 and b"built-in buffer" in lib.clg_last_error()
    rc = lib.clg_group_sum_static(0, x.data_ptr(), out.data_ptr(), 640, 65536, 7, 1.0, _lib.stream_ptr(x))
    assert rc != 0 and b"divisible" in lib.clg_last_error()


def test_group_sum_static_captured_in_a_hip_graph_replays_like_eager():
    # the documented order: address look-up once outside the capture (clg_group_sum_static_init), then the entry point
    # captured into a HIP graph (no allocation inside the capture) and replayed on new contents of the same input buffer,
    # with eager work and synchronisations between the replays; every replay equals clg_group_sum on that input
    lib = _lib.load()
    _lib.check(lib.clg_group_sum_static_init())
    torch.manual_seed(9)
    features, batch, k, tau = 2560, 128, 10, 6.5
    x = torch.rand(features, batch, device=DEV)
    out = torch.zeros(batch, k, device=DEV)
    dt = _lib.dtype_code(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _lib.check(lib.clg_group_sum_static(dt, x.data_ptr(), out.data_ptr(), features, batch, k, tau, _lib.stream_ptr(x)))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.clg_group_sum_static(dt, x.data_ptr(), out.data_ptr(), features, batch, k, tau, _lib.stream_ptr(x)))
    scratch = torch.empty(lib.clg_group_sum_scratch_bytes(dt, features, batch, k), dtype=torch.uint8, device=DEV)
    for r in range(3):
        x.copy_(torch.rand(features, batch, device=DEV))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = torch.empty(batch, k, device=DEV)
        _lib.check(lib.clg_group_sum(dt, x.data_ptr(), want.data_ptr(), scratch.data_ptr(), features, batch, k, tau, _lib.stream_ptr(x)))
        torch.cuda.synchronize()
        assert torch.equal(out, want), r
