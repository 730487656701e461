"""The benchmark's measurement aids (libnfn_mi355_probes.so, include/nfn_mi355_probes.h): launches
that finish, store nothing, and refuse bad arguments.  Not part of the path."""
import pytest

from neuralfn_amd import probes

pytestmark = pytest.mark.gpu


def test_shader_clock_probe_reports_a_plausible_clock():
    """nfn_mi355_shader_clock_probe_v1: cycles per tick of the constant clock, and its argument checks."""
    import torch
    device = torch.device("cuda:0")
    probe = probes.ShaderClockProbe(device)
    probe.start(200)
    megahertz = probe.megahertz()
    assert 100.0 < megahertz < 4000.0
    cycles, ticks, per_second = (int(v) for v in probe.result.tolist())
    assert per_second > 0 and ticks >= 200 * per_second // 1_000_000
    lib = probes.load()
    assert lib.nfn_mi355_shader_clock_probe_v1(None, 100, None) == 1
    assert lib.nfn_mi355_shader_clock_probe_v1(probe.result.data_ptr(), 0, None) == 1
    assert lib.nfn_mi355_shader_clock_probe_v1(probe.result.data_ptr(), 100001, None) == 1


def test_measurement_probes_run_and_check_their_arguments():
    """The read probes and nfn_mi355_mfma_rate_probe_v1."""
    import torch
    device = torch.device("cuda:0")
    lib = probes.load()
    assert lib.nfn_mi355_probes_abi_version() == 1
    data = torch.randint(0, 256, (1 << 21,), dtype=torch.uint8, device=device)
    half = data.numel() // 2
    sink = torch.full((4096,), -1, dtype=torch.int32, device=device)
    assert lib.nfn_mi355_read_probe_v1(data.data_ptr(), data.numel(), sink.data_ptr(), None) == 0
    assert lib.nfn_mi355_read_probe_v1(None, 0, sink.data_ptr(), None) == 0          # empty kernel
    assert lib.nfn_mi355_read_probe_v1(data.data_ptr(), 5000, sink.data_ptr(), None) == 0  # less than a piece per group
    assert lib.nfn_mi355_read_probe_v1(None, 1024, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_v1(data.data_ptr() + 4, 1024, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_v1(data.data_ptr(), -1, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_v1(data.data_ptr(), 1024, None, None) == 1
    following = data.data_ptr() + half
    for rounds in (0, 1, 8, 64):  # (more rounds than the region has pieces: the last piece again)
        assert lib.nfn_mi355_read_probe_chained_v1(data.data_ptr(), half, following, rounds,
                                                   sink.data_ptr(), None) == 0
    assert lib.nfn_mi355_read_probe_chained_v1(data.data_ptr(), half, None, 1, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_chained_v1(data.data_ptr(), 0, following, 1, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_chained_v1(data.data_ptr(), half, following, 65, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_read_probe_chained_v1(data.data_ptr(), half, following + 8, 1, sink.data_ptr(), None) == 1
    for mode in (0, 1, 2, 3):
        assert lib.nfn_mi355_mfma_rate_probe_v1(mode, 16, 8, sink.data_ptr(), None) == 0
    assert lib.nfn_mi355_mfma_rate_probe_v1(4, 16, 8, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_mfma_rate_probe_v1(0, 0, 8, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_mfma_rate_probe_v1(0, 16, 0, sink.data_ptr(), None) == 1
    assert lib.nfn_mi355_mfma_rate_probe_v1(0, 16, 8, None, None) == 1
    torch.cuda.synchronize()
    assert bool((sink == -1).all())
