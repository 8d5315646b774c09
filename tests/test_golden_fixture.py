"""The numpy oracle against vectors computed by the reference implementation itself
(tests/golden/tiny_model.npz, written by tests/golden/make_tiny_model_fixture.py).
Pins the model wiring around the attention path.  CPU only."""

import os

import numpy as np
import pytest

from oracle import model_oracle as mo

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny_model.npz")


@pytest.fixture(scope="module")
def fx():
    data = np.load(FIXTURE, allow_pickle=False)
    sd = {k[3:]: data[k] for k in data.files if k.startswith("w::")}
    cfg = dict(zip(("d_model", "n_heads", "n_layers", "d_ff", "num_features", "buffer_size", "num_components"),
                   (int(v) for v in data["cfg"])))
    return data, sd, cfg


def test_state_dict_keys_are_the_reference_ones(fx):
    _, sd, cfg = fx
    expected = {"embedder.x_embed.weight", "embedder.x_embed.bias", "embedder.y_embed.weight", "embedder.y_embed.bias",
                "embedder.marker_embed.weight", "backbone.norm.weight", "backbone.norm.bias", "head.head.0.weight",
                "head.head.0.bias", "head.head.2.weight", "head.head.2.bias", "head.mean_bias", "head.std_bias",
                "head.weight_bias", "ar_tokens"}
    for i in range(cfg["n_layers"]):
        p = f"backbone.layers.{i}"
        for a in ("attn_features", "attn_rows"):
            expected |= {f"{p}.{a}.{w}.weight" for w in ("q_proj", "k_proj", "v_proj", "out_proj")}
        expected |= {f"{p}.ff.{j}.{w}" for j in (0, 2) for w in ("weight", "bias")}
        expected |= {f"{p}.norm{j}.{w}" for j in (1, 2, 3) for w in ("weight", "bias")}
    assert set(sd) == expected


def test_oracle_log_density_per_dataset_matches_reference(fx):
    data, sd, cfg = fx
    m = mo.OracleModel(sd, cfg["n_heads"])
    ll = mo.OraclePredictor(m, "per_dataset").evaluate_joint_density(data["x_ctx"], data["y_ctx"], data["x_tgt"], data["y_tgt"])
    np.testing.assert_allclose(ll, data["ll_per_dataset"], atol=2e-5, rtol=0)


def test_oracle_log_density_shared_matches_reference(fx):
    data, sd, cfg = fx
    m = mo.OracleModel(sd, cfg["n_heads"])
    B = data["x_ctx"].shape[0]
    xc = np.repeat(data["x_ctx"][0:1], B, axis=0)
    yc = np.repeat(data["y_ctx"][0:1], B, axis=0)
    ll = mo.OraclePredictor(m, "shared").evaluate_joint_density(xc, yc, data["x_tgt"], data["y_tgt"])
    np.testing.assert_allclose(ll, data["ll_shared"], atol=2e-5, rtol=0)


@pytest.mark.parametrize("backend", ["per_dataset", "shared"])
def test_oracle_fixed_buffer_decode_matches_reference(fx, backend):
    data, sd, cfg = fx
    m = mo.OracleModel(sd, cfg["n_heads"])
    B = data["x_ctx"].shape[0]
    xc, yc = data["x_ctx"], data["y_ctx"]
    if backend == "shared":
        xc, yc = np.repeat(xc[0:1], B, axis=0), np.repeat(yc[0:1], B, axis=0)
    z = mo.OraclePredictor(m, backend).fixed_buffer_decode(xc, yc, data["x_tgt"], data["y_tgt"], ar_rule="sampling")
    np.testing.assert_allclose(z, data[f"z_decode_{backend}"], atol=2e-5, rtol=0)


def test_training_forward_matches_reference_fixture():
    """The training forward under the row mask (model.py:317-369, attention.py:86-175): the loss
    the reference computed for the fixture, with the default and with three attending chunks."""
    from oracle import model_oracle as mo

    data = np.load(FIXTURE, allow_pickle=False)
    sd = {k[3:]: data[k] for k in data.files if k.startswith("w::")}
    om = mo.OracleModel(sd, int(data["cfg"][1]))
    args = (data["x_ctx"], data["y_ctx"], data["train_x_buf"], data["train_y_buf"], data["train_x_tgt"], data["train_y_tgt"])
    loss, z = mo.training_forward(om, *args)
    assert z.shape == (3, 16, 32)
    assert abs(loss - float(data["train_loss"])) <= 2e-5
    loss3, _ = mo.training_forward(om, *args, attending_chunks=3)
    assert abs(loss3 - float(data["train_loss_attend3"])) <= 2e-5
    assert abs(loss - loss3) > 1e-4  # the attending region matters
