"""trimkv_stream_probe, the load-only kernel behind bench.py's roofline.stream_ceiling: it runs over two buffers of any
size that holds a granule, reads only whole granules, and never writes its sink."""
import pytest
import torch

from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("workgroups,extra", [(512, 0), (256, 12345), (7, 4096 * 3 + 16)])
def test_stream_probe_reads_and_leaves_its_sink_alone(workgroups, extra):
    from trimkv_amd import _lib as L
    lib = L.load()
    gran = lib.trimkv_stream_probe_granule(workgroups)
    nbytes = 5 * gran + extra                              # the tail beyond whole granules is not read
    a = torch.full((nbytes,), 0x5a, dtype=torch.uint8, device=DEV)
    b = torch.full((nbytes,), 0xc3, dtype=torch.uint8, device=DEV)
    guard = torch.zeros(64, dtype=torch.uint8, device=DEV)
    sink = guard[16:32]
    st = L.current_stream(torch.device(DEV))
    print(f"stream probe: {workgroups} workgroups, {nbytes} bytes each", flush=True)
    for _ in range(3):
        L.check(lib.trimkv_stream_probe(a.data_ptr(), b.data_ptr(), nbytes, workgroups, sink.data_ptr(), st), "trimkv_stream_probe")
    torch.cuda.synchronize()
    assert not guard.any() and bool((a == 0x5a).all()) and bool((b == 0xc3).all())
    assert lib.trimkv_stream_probe(a.data_ptr(), b.data_ptr(), gran - 1, workgroups, sink.data_ptr(), st) == -2
