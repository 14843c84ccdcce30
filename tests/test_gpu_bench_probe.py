"""GPU: the measurement aids of bench.py (bench_probe/libqtip_probe.so, a library of its own -
libqtip_hip.so exports none of it)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_instruction_rate_probe_runs_every_kind():
    """Every kind launches, fills its sink, and a full-rate instruction is measurably cheaper than
    the decode loop it is part of."""
    import bench_probe
    tlut = torch.randn(512, 2, generator=torch.Generator().manual_seed(0)).half().cuda()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    times = {}
    for name in bench_probe.KINDS:
        sink = torch.full((1024 * cus,), -1, dtype=torch.int32, device="cuda")
        bench_probe.issue(name, 20, tlut, sink)  # warm
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        bench_probe.issue(name, 400, tlut, sink)
        e1.record()
        torch.cuda.synchronize()
        times[name] = e0.elapsed_time(e1)
        assert times[name] > 0
    per_op = times["v_and_b32"] * 1e6 / (400 * bench_probe.OPS_PER_ITER * 4)
    per_item = times["decode_loop"] * 1e6 / (400 * 4)
    assert 0.2 < per_op < 20 and 50 < per_item < 2000, (per_op, per_item)
    assert times["decode_loop_valu"] < times["decode_loop"]
    with pytest.raises(ValueError):
        bench_probe.issue("v_nop", 10, tlut)
    rc = bench_probe.lib().qtip_probe_issue(55, 10, tlut.data_ptr(), sink.data_ptr(), None)
    assert rc == -1  # an unknown kind is an argument error, nothing is launched


def test_stream_read_probe_reads_every_word_once():
    import bench_probe
    for n16 in (4, 4099, 1 << 18):
        src = torch.randint(-2**31, 2**31 - 1, (n16 * 4,), dtype=torch.int32,
                            generator=torch.Generator().manual_seed(n16))
        sink = bench_probe.stream_read(src.cuda()).cpu().numpy()
        assert int(np.bitwise_xor.reduce(sink)) == int(np.bitwise_xor.reduce(src.numpy()))
