"""End to end through the host layer: the Whisper audio encoder of the reference's
examples/whisper_poc.cpp (conv stem, sinusoid-table positions, pre-norm attention / MLP
layers, final norm) run by axiom_amd/lib/whisper_encoder from a .safetensors file, against
an fp32 evaluation of the same weights written with plain torch ops on the CPU."""
import json
import math
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
BIN = ROOT / "axiom_amd" / "lib" / "whisper_encoder"


def make_weights(d_model, n_layers, ffn, n_mels, n_pos, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape, s=1.0: torch.randn(*shape, generator=g) * s
    w = {"conv1.weight": r(d_model, n_mels, 3, s=1 / math.sqrt(3 * n_mels)), "conv1.bias": r(d_model, s=0.1),
         "conv2.weight": r(d_model, d_model, 3, s=1 / math.sqrt(3 * d_model)), "conv2.bias": r(d_model, s=0.1),
         "embed_positions.weight": r(n_pos, d_model, s=0.3), "layer_norm.weight": 1 + r(d_model, s=0.1), "layer_norm.bias": r(d_model, s=0.1)}
    for i in range(n_layers):
        p = f"layers.{i}."
        for name in ("q_proj", "k_proj", "v_proj", "out_proj"):
            w[p + f"self_attn.{name}.weight"] = r(d_model, d_model, s=1 / math.sqrt(d_model))
            if name != "k_proj":  # Whisper's key projection has no bias
                w[p + f"self_attn.{name}.bias"] = r(d_model, s=0.1)
        for name in ("self_attn_layer_norm", "final_layer_norm"):
            w[p + name + ".weight"] = 1 + r(d_model, s=0.1)
            w[p + name + ".bias"] = r(d_model, s=0.1)
        w[p + "fc1.weight"], w[p + "fc1.bias"] = r(ffn, d_model, s=1 / math.sqrt(d_model)), r(ffn, s=0.1)
        w[p + "fc2.weight"], w[p + "fc2.bias"] = r(d_model, ffn, s=1 / math.sqrt(ffn)), r(d_model, s=0.1)
    return w


def reference_forward(w, mel, n_layers, heads):
    x = F.gelu(F.conv1d(mel, w["conv1.weight"], w["conv1.bias"], padding=1))
    x = F.gelu(F.conv1d(x, w["conv2.weight"], w["conv2.bias"], stride=2, padding=1)).transpose(1, 2)
    x = x + w["embed_positions.weight"][: x.shape[1]]
    B, S, Dm = x.shape
    for i in range(n_layers):
        p = f"layers.{i}."
        h = F.layer_norm(x, (Dm,), w[p + "self_attn_layer_norm.weight"], w[p + "self_attn_layer_norm.bias"])
        q = F.linear(h, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"])
        k = F.linear(h, w[p + "self_attn.k_proj.weight"])
        v = F.linear(h, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])
        split = lambda t: t.reshape(B, S, heads, Dm // heads).transpose(1, 2)
        a = torch.softmax(split(q) @ split(k).transpose(-1, -2) / math.sqrt(Dm // heads), -1) @ split(v)
        x = x + F.linear(a.transpose(1, 2).reshape(B, S, Dm), w[p + "self_attn.out_proj.weight"], w[p + "self_attn.out_proj.bias"])
        h = F.layer_norm(x, (Dm,), w[p + "final_layer_norm.weight"], w[p + "final_layer_norm.bias"])
        x = x + F.linear(F.gelu(F.linear(h, w[p + "fc1.weight"], w[p + "fc1.bias"])), w[p + "fc2.weight"], w[p + "fc2.bias"])
    return F.layer_norm(x, (Dm,), w["layer_norm.weight"], w["layer_norm.bias"])


def run_case(tmp_path, geometry, dtype, frames, tol):
    from safetensors.torch import save_file

    assert BIN.exists(), f"{BIN} is missing: run python -m axiom_amd.build --host"
    d_model, n_layers, heads, ffn, n_mels = geometry
    w = make_weights(d_model, n_layers, ffn, n_mels, 1500, seed=7)
    mel = torch.randn(1, n_mels, frames, generator=torch.Generator().manual_seed(8))
    if dtype != "f32":  # the reference sees the same rounded parameters and input
        tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
        w = {k: v.to(tdt).float() for k, v in w.items()}
        mel = mel.to(tdt).float()
    save_file({"model.encoder." + k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    save_file({"mel": mel}, str(tmp_path / "mel.safetensors"))
    out_path = tmp_path / "out.bin"
    p = subprocess.run([str(BIN), str(tmp_path / "model.safetensors"), "--layers", str(n_layers), "--heads", str(heads), "--dtype", dtype,
                        "--mel", str(tmp_path / "mel.safetensors"), "--out", str(out_path), "--repeat", "3"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    info = json.loads(p.stdout.strip().splitlines()[-1])
    print(info)
    assert info["out_shape"] == [1, frames // 2, d_model]
    got = np.fromfile(out_path, np.float32).reshape(1, frames // 2, d_model)
    with torch.no_grad():
        want = reference_forward(w, mel, n_layers, heads).numpy()
    err = np.abs(got - want)
    if tol is not None:  # fp32: the library's own 1e-4 per op, accumulated over the layers of O(1)-scaled activations
        assert err.max() < tol, err.max()
    else:  # 16-bit: every intermediate is rounded to the type; outputs are layer-normed, O(1)
        eps = 2.0**-8 if dtype == "bf16" else 2.0**-11
        assert err.max() < 40 * eps and err.mean() < 4 * eps, (err.max(), err.mean())


# whisper-tiny's encoder geometry (d_model 384, 4 layers, 6 heads, 80 mel bins), at a short
# and at the full 30 s (3000-frame) input
@pytest.mark.parametrize("dtype,frames,tol", [("f32", 200, 2e-3), ("f32", 3000, 2e-3), ("bf16", 3000, None), ("f16", 600, None)])
def test_encoder_matches_fp32_reference(tmp_path, dtype, frames, tol):
    run_case(tmp_path, (384, 4, 6, 1536, 80), dtype, frames, tol)


# one layer at whisper-large's width (d_model 1280, 20 heads of 64, ffn 5120, 128 mel bins) over the full
# 3000 frames: the shapes of the Whisper-style block the benchmarks time ([1, 1500, 1280], 20 x 64)
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_large_width_layer_matches_fp32_reference(tmp_path, dtype):
    run_case(tmp_path, (1280, 1, 20, 5120, 128), dtype, 3000, None)
