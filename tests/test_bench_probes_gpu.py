"""The benchmark's measurement aids (``libditango_probes.so`` through ``bench_probes.py``): each probe runs,
leaves its inputs alone and refuses bad arguments without a launch.  They are not part of the drop-in library."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def probes():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import bench_probes
    bench_probes.load_library()
    return bench_probes


def test_read_probe_and_its_argument_checks(probes):
    """The bandwidth yardstick reads its streams and writes nothing; bad arguments are refused without a launch."""
    bufs = [torch.full((1000, 64), 3, dtype=torch.int32, device="cuda") for _ in range(11)]    # 256 000 bytes each
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    probes.hbm_read_probe(bufs, sink)
    torch.cuda.synchronize()
    assert int(sink.item()) == 0 and all(int(b.sum().item()) == 3 * 64000 for b in bufs)
    with pytest.raises(probes.ProbeError):
        probes.hbm_read_probe(bufs + [bufs[0][:500]], sink)
    with pytest.raises(probes.ProbeError):
        probes.hbm_read_probe(bufs * 6, sink)                     # 66 streams: more than one launch takes


def test_mfma_probe_runs_and_checks_its_arguments(probes):
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    flop = probes.mfma_probe(64, 16, sink)
    torch.cuda.synchronize()
    assert flop == 64 * 8 * 4 * 16 * 32768.0 and float(sink) == 0.0
    for bad in ((0, 16), (64, 0), (-1, 4), (64, 6)):
        with pytest.raises(probes.ProbeError):
            probes.mfma_probe(*bad, sink)


def test_coissue_probe_runs_and_checks_its_arguments(probes):
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    for D in (64, 128):
        for with_softmax in (False, True):
            flop = probes.coissue_probe(64, 16, D, with_softmax, sink)
            torch.cuda.synchronize()
            assert flop == 64 * 4 * 4 * 16 * 32768.0 and float(sink) == 0.0
    for bad in ((0, 16, 128), (64, 0, 128), (64, 6, 64), (64, 16, 96)):
        with pytest.raises(probes.ProbeError):
            probes.coissue_probe(*bad, True, sink)


def test_empty_launch_runs_and_checks_its_arguments(probes):
    probes.empty_launch(3333, 256)
    torch.cuda.synchronize()
    for bad in ((0, 256), (10, 0), (10, 100), (10, 2048)):
        with pytest.raises(probes.ProbeError):
            probes.empty_launch(*bad)
