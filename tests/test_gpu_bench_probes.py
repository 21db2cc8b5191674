"""The measurement aids of bench.py (bench_probes/, not part of the product library) do what bench.py assumes."""
import pytest
import torch

import bench_probes as P

pytestmark = pytest.mark.gpu


def test_gather_probe_runs_and_checks_its_arguments(gpu):
    """The measurement aid reads and writes nothing a caller can see; bad arguments are refused."""
    buf = torch.arange(1 << 18, dtype=torch.int32, device=gpu)
    before = buf.clone()
    assert P.gather_probe(buf, unit_bytes=64, iters=3, blocks=8) == 8 * 256 * 4 * 3
    assert P.gather_probe(buf, unit_bytes=256, iters=1, blocks=1) == 1024
    assert P.gather_probe(buf, unit_bytes=128, iters=2, blocks=2, lanes_per_unit=8) == 2 * 256 * 4 * 2 // 8
    with pytest.raises(RuntimeError):
        P.gather_probe(buf, unit_bytes=64, lanes_per_unit=8)        # 8 lanes x 16 bytes do not fit 64
    torch.cuda.synchronize()
    assert torch.equal(buf, before)
    with pytest.raises(RuntimeError):
        P.gather_probe(buf, unit_bytes=48)
    with pytest.raises(RuntimeError):
        P.gather_probe(buf[:8], unit_bytes=64)


def test_atomic_probe_adds_what_it_says(gpu):
    """The measurement aid for atomics: every add is 1.0f, so the scratch sums to the number of adds."""
    scratch = torch.zeros(1 << 16, dtype=torch.float32, device=gpu)
    adds, requests = P.atomic_probe(scratch, run_floats=16, iters=5, blocks=3)
    assert adds == 3 * 256 * 5 and requests == adds // 16
    assert float(scratch.double().sum()) == adds
    adds, requests = P.atomic_probe(scratch, run_floats=1, iters=2, blocks=2)
    assert requests == adds
    with pytest.raises(RuntimeError):
        P.atomic_probe(scratch, run_floats=3)
    with pytest.raises(RuntimeError):
        P.atomic_probe(scratch[1:17], run_floats=16)       # not 64-byte aligned
