"""The counterparts of the reference's benchmark scripts (benchmarks/benchmark_layer_norm.py,
benchmark_instance_norm.py) as a tested artefact: one shape of each table goes through the
scripts' own code path (same layer construction, same train step), timed with one warm-up and
one repeat, and the fused column's outputs are checked against the torch column's."""
import pytest

pytestmark = pytest.mark.gpu


def _check(fused, native):
    import torch

    y, dx, dg, db = fused
    yr, dxr, dgr, dbr = native
    assert torch.allclose(y.float(), yr.float(), rtol=1e-2, atol=1e-2)
    assert torch.allclose(dx.float(), dxr.float(), rtol=1e-2, atol=1e-2)
    # parameter gradients: float32 sums on one side, torch's reduction of fp16 terms on the other
    scale = float(dgr.float().abs().max()) + 1.0
    assert float((dg.float() - dgr.float()).abs().max()) <= 2e-2 * scale
    assert float((db.float() - dbr.float()).abs().max()) <= 2e-2 * (float(dbr.float().abs().max()) + 1.0)


def test_layer_norm_benchmark_script():
    from atex_amd.benchmarks import benchmark_layer_norm as B

    shape = (100000, 1000)
    assert shape in B.SHAPES
    print(f"benchmark_layer_norm shape={shape}", flush=True)
    rows = B.run(shapes=[shape], warmup=1, repeat=1)
    assert len(rows) == 1 and rows[0]["fused_ms"] > 0 and rows[0]["torch_ms"] > 0
    _check(B.outputs(shape, True), B.outputs(shape, False))


@pytest.mark.parametrize("channel_last", [True, False])
def test_instance_norm_benchmark_script(channel_last):
    from atex_amd.benchmarks import benchmark_instance_norm as B

    s = (8, 32, 64)
    assert s in B.SHAPES
    print(f"benchmark_instance_norm shape={s} channel_last={channel_last}", flush=True)
    rows = B.run(shapes=[s], warmup=1, repeat=1)
    assert len(rows) == 2 and all(r["fused_ms"] > 0 and r["torch_ms"] > 0 for r in rows)
    shape = B.expand(s, channel_last)
    _check(B.outputs(shape, channel_last, True), B.outputs(shape, channel_last, False))
