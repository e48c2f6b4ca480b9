"""The loader for coffin's pre-quantised directories (quantized_load.py:46-51,186-330 describe the
formats).  The directories here are written by this test in the layout the reference's writers
produce (tools/quant_disk.py, tools/quant_disk_w4a8.py:225-286): per shard a safetensors file,
``<key>#scale`` beside each quantised tensor, ``quant_index.json`` with kind / shapes / shard /
scale_key per tensor."""

from __future__ import annotations

import hashlib
import json

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from coffin_amd import quantized_load as ql
from coffin_amd import synth
from coffin_amd.weights import QWeight, W4A8Weight

P = "model.language_model.layers.0."


def _write_int8_dir(tmp_path, with_config=True):
    g = synth.generator()
    q1, q2 = synth.int8_weight(24, 32, g), synth.int8_weight(40, 16, g)
    norm = torch.randn(32, generator=g).to(torch.bfloat16)
    tensors = {P + "mlp.up_proj.weight": q1.wq.t().contiguous(), P + "mlp.up_proj.weight#scale": q1.scale,
               P + "input_layernorm.weight": norm}
    save_file(tensors, str(tmp_path / "quant-00001-of-00002.safetensors"))
    save_file({"lm_head.weight": q2.wq.t().contiguous(), "lm_head.weight#scale": q2.scale,
               "model.visual.patch.weight": torch.zeros(4)}, str(tmp_path / "quant-00002-of-00002.safetensors"))
    index = {"format": ql.FORMAT_INT8, "weight_dtype": "bfloat16", "tensors": {
        P + "mlp.up_proj.weight": {"kind": "q8", "shape": [32, 24], "K": 32, "N": 24,
                                   "scale_key": P + "mlp.up_proj.weight#scale",
                                   "shard": "quant-00001-of-00002.safetensors"},
        P + "input_layernorm.weight": {"kind": "dense", "shape": [32], "shard": "quant-00001-of-00002.safetensors"},
        "lm_head.weight": {"kind": "q8", "shape": [16, 40], "K": 16, "N": 40, "scale_key": "lm_head.weight#scale",
                           "shard": "quant-00002-of-00002.safetensors"},
        "model.visual.patch.weight": {"kind": "dense", "shape": [4], "shard": "quant-00002-of-00002.safetensors"}}}
    if with_config:
        (tmp_path / "config.json").write_text('{"hidden_size": 32}')
        index["source_config_sha256"] = hashlib.sha256((tmp_path / "config.json").read_bytes()).hexdigest()
    (tmp_path / ql.INDEX_NAME).write_text(json.dumps(index))
    return q1, q2, norm, index


def test_int8_directory_comes_back_as_row_major_qweights(tmp_path, orc):
    q1, q2, norm, _ = _write_int8_dir(tmp_path)
    assert ql.is_quantized_dir(tmp_path) and not ql.is_quantized_dir(tmp_path / "nowhere")
    sd = ql.load(tmp_path, device="cpu")
    assert set(sd) == {P + "mlp.up_proj.weight", P + "input_layernorm.weight", "lm_head.weight"}   # no vision tower
    w = sd[P + "mlp.up_proj.weight"]
    assert isinstance(w, QWeight) and (w.n, w.k) == (24, 32) and w.wq.is_contiguous()
    assert (w.wq == q1.wq).all() and (w.scale == q1.scale).all()            # [K,N] on disk -> [N,K] rows
    assert (sd["lm_head.weight"].wq == q2.wq).all()
    assert (sd[P + "input_layernorm.weight"].view(torch.int16) == norm.view(torch.int16)).all()
    # quant=False hands out the dequantised matrix in the recorded dtype (one rounding, int8_weights.py:359)
    dense = ql.load(tmp_path, device="cpu", quant=False, keep=lambda k: k.startswith("lm_head"))
    assert set(dense) == {"lm_head.weight"} and dense["lm_head.weight"].dtype == torch.bfloat16
    want = orc.qweight_dequant_bf16(q2.wq.numpy(), q2.scale.numpy())
    assert (dense["lm_head.weight"].view(torch.int16).numpy().view(np.uint16) == want).all()


def test_w4a8_directory_comes_back_in_the_contract_layout(tmp_path, orc):
    g = synth.generator()
    w = synth.int4_weight(24, 256, g)
    key = P + "self_attn.q_proj.weight"
    save_file({key: w.packed, key + "#scale": w.scale}, str(tmp_path / "quant-00001-of-00001.safetensors"))
    index = {"format": ql.FORMAT_W4A8, "weight_dtype": "bfloat16", "group_size": 128, "tensors": {
        key: {"kind": "q4", "shape": [24, 256], "n": 24, "k": 256, "group_size": 128, "groups": 2,
              "packed_shape": [128, 24], "scale_shape": [2, 24], "scale_key": key + "#scale",
              "shard": "quant-00001-of-00001.safetensors"}}}
    (tmp_path / ql.INDEX_NAME).write_text(json.dumps(index))
    got = ql.load(tmp_path, device="cpu")[key]
    assert isinstance(got, W4A8Weight) and (got.n, got.k, got.group_size) == (24, 256, 128)
    assert (got.packed == w.packed).all() and (got.scale == w.scale).all()
    dense = ql.load(tmp_path, device="cpu", quant=False)[key]
    want = orc.bf16_from_f32(orc.w4_dequant_f32(w.packed.numpy(), w.scale.numpy(), 256, 128))
    assert (dense.view(torch.int16).numpy().view(np.uint16) == want).all()
    # a fused expert stack is refused, not handed out as if it were a projection
    index["tensors"][key]["kind"] = "q4-moe"
    (tmp_path / ql.INDEX_NAME).write_text(json.dumps(index))
    with pytest.raises(ValueError, match="expert"):
        ql.load(tmp_path, device="cpu")


def test_index_and_shards_are_checked_before_anything_is_built(tmp_path):
    _, _, _, index = _write_int8_dir(tmp_path)
    key = P + "mlp.up_proj.weight"

    def rewrite(mutate):
        bad = json.loads(json.dumps(index))
        mutate(bad)
        (tmp_path / ql.INDEX_NAME).write_text(json.dumps(bad))

    rewrite(lambda i: i.__setitem__("format", "coffin-int8-kn-v0"))
    with pytest.raises(ValueError, match="unsupported quantized format"):
        ql.read_index(tmp_path)
    rewrite(lambda i: i["tensors"][key].__setitem__("shape", [24, 32]))
    with pytest.raises(ValueError, match="index says shape"):
        ql.load(tmp_path, device="cpu")
    rewrite(lambda i: i["tensors"][key].__setitem__("scale_key", key + "#nope"))
    with pytest.raises(ValueError, match="no scale tensor"):
        ql.load(tmp_path, device="cpu")
    rewrite(lambda i: i["tensors"][key].__setitem__("shard", "quant-00009-of-00002.safetensors"))
    with pytest.raises(FileNotFoundError):
        ql.load(tmp_path, device="cpu")
    rewrite(lambda i: None)
    with pytest.raises(ValueError, match="asked for"):
        ql.load(tmp_path, device="cpu", weight_dtype=torch.float16)
    with pytest.raises(ValueError, match="no tensor under"):
        ql.load(tmp_path, device="cpu", prefixes=("model.nothing.",))
    (tmp_path / "config.json").write_text('{"hidden_size": 64}')
    with pytest.raises(ValueError, match="mixes two checkpoints"):
        ql.load(tmp_path, device="cpu")
