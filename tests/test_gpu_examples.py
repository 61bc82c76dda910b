"""The two toy models (Conv2D -> norm, sum loss, one training step) run with the fused layers
and with torch's own norms from the same seed: every gradient must agree.  Shapes are those
of the reference's examples (sample_layerN.py:15, sample_instanceN.py:16)."""
import pytest

pytestmark = pytest.mark.gpu


def _compare(mod):
    import torch

    torch.manual_seed(0)
    fused = mod.build_model(True)
    torch.manual_seed(0)
    plain = mod.build_model(False)
    # same convolution weights in both (the norm weights start at gamma = 1, beta = 0)
    plain.conv2d.load_state_dict(fused.conv2d.state_dict())
    data = torch.randn(mod.N, mod.H, mod.W, mod.C, device="cuda")
    from atex_amd.examples.toy import train_step
    gf = train_step(fused, data)
    gp = train_step(plain, data)
    torch.cuda.synchronize()
    assert torch.allclose(fused(data), plain(data), rtol=1e-4, atol=1e-5)
    for name in ("conv2d.conv.weight", "conv2d.conv.bias"):
        assert torch.allclose(gf[name], gp[name], rtol=1e-3, atol=2e-4), name
    # the norm's own weights: gamma / beta of the fused layer vs weight / bias of torch's
    assert torch.allclose(gf["norm.gamma"].reshape(-1), gp["norm.inner.weight"].reshape(-1), rtol=1e-4, atol=1e-4)
    assert torch.allclose(gf["norm.beta"].reshape(-1), gp["norm.inner.bias"].reshape(-1), rtol=1e-4, atol=1e-4)


def test_sample_layer_norm_model():
    from atex_amd.examples import sample_layerN
    _compare(sample_layerN)
    assert set(sample_layerN.main(["--nvops"])) >= {"norm.gamma", "norm.beta"}


def test_sample_instance_norm_model():
    from atex_amd.examples import sample_instanceN
    _compare(sample_instanceN)
    assert set(sample_instanceN.main(["--nvops"])) >= {"norm.gamma", "norm.beta"}
