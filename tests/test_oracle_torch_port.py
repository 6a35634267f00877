"""Pins of ``oracle/torch_port.py`` (the torch-CPU form of the dequantize-then-attend path that
``bench.py`` times as a CPU baseline): against what the reference itself wrote for the golden
per-head layers, and against the NumPy oracle on a larger seeded layer."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from oracle import torch_port as TP
from rdkv_amd import synth
from tests.helpers import golden_to_oracle_layer, load_golden


@pytest.mark.parametrize("name", ["perhead_d128_a", "perhead_d128_b"])
def test_torch_port_matches_reference_outputs(name):
    g = load_golden(name)
    pl = golden_to_oracle_layer(g, "pl")
    tl = TP.TorchLayer(pl, g["new_v_only"])
    k_hat = TP.unpack_k(tl).numpy()
    assert np.array_equal(k_hat.view(np.uint16), g["K_hat"][0].view(np.uint16)), "K_hat bits"
    v_hat = TP.unpack_v(tl).numpy()
    t_v = g["V_zone_a"].shape[1]
    assert np.array_equal(v_hat[:, :t_v].view(np.uint16), g["V_zone_a"].view(np.uint16)), "V zone A bits"
    assert np.array_equal(v_hat[:, t_v:].view(np.uint16), g["new_v_only"][0].view(np.uint16)), "V zone B bits"
    out, weights, scores = TP.decode_attn(torch.from_numpy(g["q"]), tl)
    valid = np.isfinite(g["pl.softmax_mask"])
    np.testing.assert_allclose(scores.numpy()[valid], g["scores"][valid], rtol=0, atol=2e-6)
    np.testing.assert_allclose(weights.numpy(), g["weights"], rtol=0, atol=2e-7)
    np.testing.assert_allclose(out.numpy(), g["out"], rtol=0, atol=2e-6)


def test_torch_port_matches_numpy_oracle_on_a_config_shaped_layer():
    cfg = synth.scaled(synth.CONFIGS[1], context=1800, layers=1)
    vb, kb, oc = synth.layer_allocation(cfg, 0)
    K, V, q = synth.layer_data(cfg, 0, "cpu", outliers=oc)
    pl, nvo = O.pack_layer_per_head(K.numpy(), V.numpy(), vb.numpy(), kb.numpy(), cfg.G)
    exp_out, _, exp_w = O.decode_attn_ref(q.numpy(), pl, nvo)
    tl = TP.TorchLayer(pl, nvo)
    assert np.array_equal(TP.unpack_k(tl).numpy().view(np.uint16), O.unpack_k_mixed(pl, D=128)[0].view(np.uint16))
    out, weights, _ = TP.decode_attn(q, tl)
    # (fp32 on both sides, other summation orders: a few units in the last place of a weight)
    np.testing.assert_allclose(weights.numpy(), exp_w, rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(out.numpy(), exp_out, rtol=0, atol=5e-6)
