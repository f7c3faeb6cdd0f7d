"""Timing helpers run and return sane numbers (not a benchmark)."""
import pytest

from reef_amd import binding as B
from reef_amd.modelgen import nets
from tests.helpers import write_model

pytestmark = pytest.mark.gpu


def test_time_kernel_and_model(tmp_path):
    g = nets.resnet(18, image=(3, 64, 64), classes=10, name="tiny")
    d = write_model(g, tmp_path)
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    us = exe.time_kernel(1, warmup=2, iters=10)
    assert 0.5 < us < 5000
    lat, dev = exe.time_model(warmup=2, iters=5)
    assert (lat > 0).all() and (dev > 0).all()
