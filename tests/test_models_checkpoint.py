"""The pieces either side of the hot path: model mirrors (embed / readout, state-dict layout of
gridnet/scripts/train_mnist.py:14-65, train_imagenet.py:17-87, gridnet/__init__.py:102-121) and
the web checkpoint blob (gridnet/scripts/convert_to_web.py:33-71, web/ts/checkpoint.ts:28-99)."""

import json
import struct

import numpy as np
import pytest
import torch

from gridnet_amd.checkpoint import (pack_float16, read_web_checkpoint, unpack_float16,
                                    write_web_checkpoint)


def test_float16_packing_known_answers():
    # worked by hand from the converter's bit formula: sign | (exp+15)&31 << 10 | frac >> 13
    v = np.array([1.0, -2.5, 0.5, 65504.0], dtype=np.float32)
    assert [int(h) for h in pack_float16(v)] == [0x3C00, 0xC100, 0x3800, 0x7BFF]
    # 1/3 = 0x3EAAAAAB: exp -2, frac 0x2AAAAB -> truncated (not rounded) to 0x155
    assert int(pack_float16(np.array([1 / 3], dtype=np.float32))[0]) == (13 << 10) | 0x155
    np.testing.assert_array_equal(unpack_float16(np.array([0x3C00, 0xC100, 0x3800, 0x7BFF])),
                                  np.array([1.0, -2.5, 0.5, 65504.0], dtype=np.float32))


def test_float16_packing_keeps_the_formats_quirk_for_tiny_values():
    # exponents below -15 are clamped to -15 and the reader has no subnormals or zero:
    # 0.0 -> 0x0000 -> 2^-15; 1e-6 (0x358637BD, exp -20, frac>>13 = 0x31) -> 2^-15 * (1 + 49/1024)
    h = pack_float16(np.array([0.0, 1e-6, -0.0], dtype=np.float32))
    assert [int(x) for x in h] == [0x0000, 0x0031, 0x8000]
    back = unpack_float16(h)
    assert back[0] == 2.0 ** -15 and back[2] == -(2.0 ** -15)
    assert back[1] == np.float32(2.0 ** -15 * (1 + 49 / 1024))


def test_checkpoint_blob_layout_and_round_trip(tmp_path):
    state = {"init_in": torch.arange(8, dtype=torch.float32).reshape(2, 2, 2) - 3.5,
             "norm.weight": torch.tensor([1.0, -2.5])}
    path = tmp_path / "ckpt.bin"
    write_web_checkpoint(path, state, activation="silu", inner_iters=3, outer_iters=5,
                         outer_residual=True, precision=32)
    blob = path.read_bytes()
    (size,) = struct.unpack("<I", blob[:4])
    meta = json.loads(blob[4:4 + size])
    assert meta == {"params": [["init_in", [2, 2, 2]], ["norm.weight", [2]]], "precision": 32,
                    "config": {"activation": "silu", "innerIters": 3, "outerIters": 5,
                               "outerResidual": True}}
    assert blob[4 + size:] == struct.pack("<10f", *(list(np.arange(8) - 3.5) + [1.0, -2.5]))
    got, config, precision = read_web_checkpoint(path)
    assert precision == 32 and config["innerIters"] == 3
    assert list(got) == list(state)
    for k in state:
        assert torch.equal(got[k], state[k])


def test_checkpoint_precision_16_round_trip(tmp_path):
    g = torch.Generator().manual_seed(0)
    state = {"w": torch.randn(3, 4, 5, generator=g), "b": torch.randn(7, generator=g) * 30}
    path = tmp_path / "ckpt16.bin"
    write_web_checkpoint(path, state, precision=16)
    blob = path.read_bytes()
    (size,) = struct.unpack("<I", blob[:4])
    assert len(blob) == 4 + size + 2 * (60 + 7)
    got, _, precision = read_web_checkpoint(path)
    assert precision == 16
    for k, v in state.items():
        big = v.abs() >= 2.0 ** -14
        # truncation of 13 mantissa bits: relative error below 2^-10, never above the value
        rel = ((got[k] - v).abs() / v.abs())[big]
        assert (rel < 2.0 ** -10).all()
        assert (got[k].abs() <= v.abs())[big].all()


def test_checkpoint_rejects_inconsistent_metadata(tmp_path):
    path = tmp_path / "bad.bin"
    meta = json.dumps({"params": [["w", [3]]], "precision": 32, "config": {}}).encode()
    path.write_bytes(struct.pack("<I", len(meta)) + meta + struct.pack("<4f", 1, 2, 3, 4))
    with pytest.raises(ValueError):
        read_web_checkpoint(path)


MNIST_KEYS = {"init_in": (32, 32, 32), "network.weight": (27, 32, 32, 32),
              "network.bias": (32, 32, 32), "network.residual_scale": (32, 32, 32),
              "norm.weight": (32, 32, 32), "norm.bias": (32, 32, 32),
              "readout.norm.weight": (1024,), "readout.norm.bias": (1024,),
              "readout.proj.weight": (10, 1024), "readout.proj.bias": (10,)}


def test_mnist_model_state_dict_layout():
    from gridnet_amd.models import MnistGridModel

    m = MnistGridModel(2, 2, 1.0, 1.0, "silu", False, 0.0, torch.device("cpu"))
    assert {k: tuple(v.shape) for k, v in m.state_dict().items()} == MNIST_KEYS
    gated = MnistGridModel(2, 2, 1.0, 1.0, "tanh", True, 2.5, torch.device("cpu"))
    sd = gated.state_dict()
    assert tuple(sd["network.weight"].shape) == (27, 2, 32, 32, 32)
    assert tuple(sd["network.bias"].shape) == (2, 32, 32, 32)
    assert (sd["network.bias"][1] == 2.5).all() and (sd["network.bias"][0] == 0).all()
    assert "network.residual_scale" not in sd


def test_imagenet_model_state_dict_layout_and_embed():
    from gridnet_amd.models import ImageNetGridModel

    kw = dict(inner_iters=2, outer_iters=3, outer_residual=False, init_scale=1.0,
              residual_scale=0.5, emb_channels=4, grid_size=16, activation="leaky_relu",
              device=torch.device("cpu"))
    m = ImageNetGridModel(separate_params=False, **kw)
    shapes = {k: tuple(v.shape) for k, v in m.state_dict().items()}
    assert shapes["patch_emb.weight"] == (4, 3, 16, 16) and shapes["patch_emb.bias"] == (4,)
    assert shapes["network.weight"] == (27, 16, 16, 16)
    assert shapes["readout.proj.weight"] == (1000, 256)
    assert (m.state_dict()["network.residual_scale"] == 0.5).all()
    sep = ImageNetGridModel(separate_params=True, **kw)
    assert {f"networks.{i}.weight" for i in range(3)} <= set(sep.state_dict())
    # embedding: the first emb_channels K-layers are the patch embedding, the rest the learned grid
    images = torch.randn(2, 3, 256, 256)
    acts = m.embed(images)
    assert acts.shape == (2, 16, 16, 16)
    assert torch.equal(acts[:, :, :, 4:], m.init_in[None, :, :, 4:].expand(2, -1, -1, -1))
    torch.testing.assert_close(acts[:, :, :, :4], m.patch_emb(images).permute(0, 2, 3, 1))


def test_mnist_embed_and_readout_on_cpu():
    from gridnet_amd.models import MnistGridModel, Readout

    m = MnistGridModel(1, 1, 1.0, 1.0, "silu", False, 0.0, torch.device("cpu"))
    batch = torch.rand(3, 1, 28, 28)
    acts = m.embed(batch)
    assert torch.equal(acts[:, 2:-2, 2:-2, 0], batch.reshape(3, 28, 28))
    assert torch.equal(acts[:, :, :, 1:], m.init_in[None, :, :, 1:].expand(3, -1, -1, -1))
    r = Readout((4, 5, 6), 7, torch.device("cpu"), output_layers=2)
    x = torch.randn(2, 4, 5, 6)
    want = torch.nn.functional.linear(
        torch.nn.functional.layer_norm(x[:, :, :, -2:].flatten(1), (40,), r.norm.weight, r.norm.bias),
        r.proj.weight, r.proj.bias)
    torch.testing.assert_close(r(x), want)


@pytest.mark.gpu
def test_mnist_model_forward_backward_matches_oracle_composition():
    """Logits and gradients of the whole model on the GPU against embed -> oracle body -> readout
    in fp64 on the CPU with the same parameters."""
    from gridnet_amd.models import MnistGridModel
    from oracle.network import network_forward

    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    m = MnistGridModel(2, 2, 1.0, 1.0, "leaky_relu", False, 0.0, dev)
    with torch.no_grad():
        m.network.bias.normal_(0, 0.1)
        m.norm.weight.normal_(1, 0.1)
        m.norm.bias.normal_(0, 0.1)
    batch = torch.rand(2, 1, 28, 28)
    target = torch.tensor([3, 7])
    print("mnist model on the GPU", flush=True)
    logits = m(batch.to(dev))
    loss = torch.nn.functional.cross_entropy(logits, target.to(dev))
    loss.backward()

    ref = {k: v.detach().cpu().double().requires_grad_(True) for k, v in m.state_dict().items()}
    init = ref["init_in"][None].repeat(2, 1, 1, 1)
    init[:, 2:-2, 2:-2, 0] = batch.reshape(2, 28, 28).double()
    h = network_forward(ref["network.weight"], ref["network.bias"], ref["network.residual_scale"],
                        ref["norm.weight"], ref["norm.bias"], init, 2, 2, 8, "leaky_relu", False)
    feat = torch.nn.functional.layer_norm(h[:, :, :, -1:].flatten(1), (1024,),
                                          ref["readout.norm.weight"], ref["readout.norm.bias"])
    want = torch.nn.functional.linear(feat, ref["readout.proj.weight"], ref["readout.proj.bias"])
    torch.nn.functional.cross_entropy(want, target).backward()

    from helpers import assert_close
    assert_close(logits, want, what="logits")
    params = dict(m.named_parameters())
    for k in ("init_in", "network.weight", "network.bias", "network.residual_scale", "norm.weight",
              "norm.bias", "readout.proj.weight"):
        assert_close(params[k].grad, ref[k].grad, what=f"d{k}")
