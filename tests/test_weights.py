"""The safetensors reader and writer, the loader's one error, dtype rules and the random-weights mode (no GPU)."""
import json
import struct

import pytest
import torch

from dinfer_amd.config.qwen3 import Qwen3Config
from dinfer_amd.config.registry import get_architecture
from dinfer_amd.parts import DecoderModel
from dinfer_amd.weights import (SafetensorsDir, WeightError, WeightFileError, WeightLoader, write_random_model,
                                write_safetensors)
from tiny_configs import CONFIGS


def model_for(name):
    cfg = Qwen3Config.from_dict(CONFIGS[name][0])
    return cfg, DecoderModel(get_architecture(cfg.ARCHITECTURE).build_spec(cfg))


def rewrite(model_dir, change):
    """Reads all tensors of the folder, lets `change` edit the dict, writes it back."""
    src = SafetensorsDir(model_dir)
    t = {n: src.read(n) for n in src.names()}
    src.close()
    change(t)
    write_safetensors(model_dir / "model.safetensors", t)


def test_writer_is_read_by_the_safetensors_package_and_back(tmp_path):
    from safetensors.torch import load_file, save_file
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b.c": torch.arange(7, dtype=torch.int64), "z": torch.randn(2, 2, 2),
         "empty": torch.zeros(0, 4)}
    write_safetensors(tmp_path / "x.safetensors", t, metadata={"k": "v"})
    back = load_file(str(tmp_path / "x.safetensors"))
    assert set(back) == set(t) and all(torch.equal(back[k], t[k]) for k in t)
    (tmp_path / "second").mkdir()
    save_file(t, str(tmp_path / "second" / "model.safetensors"))
    src = SafetensorsDir(tmp_path / "second")
    assert src.names() == sorted(t) and all(torch.equal(src.read(k), t[k]) for k in t)
    assert src.info("a").dtype_name == "BF16" and tuple(src.info("z").shape) == (2, 2, 2)


def test_several_files_form_one_index(tmp_path):
    write_safetensors(tmp_path / "model-00002.safetensors", {"b": torch.ones(2)})
    write_safetensors(tmp_path / "model-00001.safetensors", {"a": torch.zeros(3)})
    src = SafetensorsDir(tmp_path)
    assert src.names() == ["a", "b"] and "a" in src and "c" not in src


def test_broken_files(tmp_path):
    with pytest.raises(WeightFileError, match="no .*safetensors"):
        SafetensorsDir(tmp_path)
    (tmp_path / "m.safetensors").write_bytes(b"\x01\x02")
    with pytest.raises(WeightFileError, match="too short"):
        SafetensorsDir(tmp_path)
    (tmp_path / "m.safetensors").write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(WeightFileError, match="header length"):
        SafetensorsDir(tmp_path)
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    (tmp_path / "m.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(WeightFileError, match="w"):
        SafetensorsDir(tmp_path)
    hdr = json.dumps({"w": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    (tmp_path / "m.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 4)
    with pytest.raises(WeightFileError, match="unsupported dtype"):
        SafetensorsDir(tmp_path)


def test_expected_names_tied_and_untied():
    _, tied = model_for("A")
    exp, optional = tied.expected_tensors()
    assert "lm_head.weight" not in exp and optional == {"lm_head.weight"}
    assert exp["model.embed_tokens.weight"].shape == (256, 64)
    assert exp["model.layers.1.self_attn.q_norm.weight"].shape == (16,)
    _, untied = model_for("B")
    exp, optional = untied.expected_tensors()
    assert exp["lm_head.weight"].shape == (512, 96) and not optional
    assert exp["model.layers.2.self_attn.k_proj.weight"].shape == (64, 96)   # kv_heads * head_dim x hidden
    assert exp["model.layers.0.mlp.down_proj.weight"].shape == (96, 224)
    assert len(exp) == 2 + 1 + 3 * 11


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg, model = model_for("B")
    write_random_model(cfg, tmp_path, seed=1)

    def change(t):
        del t["model.layers.1.mlp.up_proj.weight"], t["lm_head.weight"]
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
        t["model.norm.weight"] = torch.zeros(95)
        t["model.layers.2.self_attn.o_proj.weight"] = torch.zeros(256, 96)   # transposed
        t["model.layers.0.input_layernorm.weight"] = torch.zeros(96, dtype=torch.int32)

    rewrite(tmp_path, change)
    loader = WeightLoader(tmp_path, "cpu", torch.float32)
    with pytest.raises(WeightError) as e:
        model.load(loader)
    err = e.value
    assert err.missing == ["lm_head.weight", "model.layers.1.mlp.up_proj.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert sorted(n for n, *_ in err.wrong_shape) == ["model.layers.2.self_attn.o_proj.weight", "model.norm.weight"]
    msg = str(err)
    for needle in ("missing tensors", "unexpected tensors", "wrong shapes", "[256, 96]", "expected [96, 256]",
                   "input_layernorm.weight is stored as I32"):
        assert needle in msg


def test_tied_head_uses_the_file_head_when_present(tmp_path):
    cfg, model = model_for("A")
    write_random_model(cfg, tmp_path, seed=1)
    model.load(WeightLoader(tmp_path, "cpu", torch.float32))
    assert model.head.weight.data_ptr() == model.embed.data_ptr()      # one buffer for both
    rewrite(tmp_path, lambda t: t.__setitem__("lm_head.weight", torch.full((256, 64), 0.5)))
    _, model2 = model_for("A")
    model2.load(WeightLoader(tmp_path, "cpu", torch.float32))
    assert model2.head.weight.data_ptr() != model2.embed.data_ptr() and float(model2.head.weight[0, 0]) == 0.5


def test_dtype_rules(tmp_path):
    """bf16 storage stays bf16 (float32 on the 32-bit path); a tensor stored in 32-bit stays so unless it is
    a matrix-product operand; integer tables become int32."""
    write_safetensors(tmp_path / "m.safetensors", {
        "w16": torch.randn(4, 4).to(torch.bfloat16), "g32": torch.randn(4), "h16": torch.randn(4).to(torch.float16),
        "table": torch.arange(5, dtype=torch.int64)})
    bf = WeightLoader(tmp_path, "cpu", torch.bfloat16)
    assert bf.fetch("w16").dtype == torch.bfloat16 and bf.fetch("h16").dtype == torch.bfloat16
    assert bf.fetch("g32").dtype == torch.float32 and bf.fetch("g32", compute=True).dtype == torch.bfloat16
    assert bf.fetch("table").dtype == torch.int32 and bf.fetch("table").tolist() == [0, 1, 2, 3, 4]
    f32 = WeightLoader(tmp_path, "cpu", torch.float32)
    assert f32.fetch("w16").dtype == torch.float32 and torch.equal(f32.fetch("w16"), bf.fetch("w16").float())
    with pytest.raises(WeightError, match="nope"):
        bf.fetch("nope")


def test_fused_operands_keep_row_order(tmp_path):
    """q|k|v and gate|up are concatenated by rows in that order (model.rs:141-165, nn.rs:288-302)."""
    cfg, model = model_for("B")
    write_random_model(cfg, tmp_path, seed=5, dtype="float32")
    model.load(WeightLoader(tmp_path, "cpu", torch.float32))
    src = SafetensorsDir(tmp_path)
    p = "model.layers.1."
    qkv = model.blocks[1].mixer.qkv.weight
    assert torch.equal(qkv[:256], src.read(p + "self_attn.q_proj.weight"))
    assert torch.equal(qkv[256:320], src.read(p + "self_attn.k_proj.weight"))
    assert torch.equal(qkv[320:], src.read(p + "self_attn.v_proj.weight"))
    gu = model.blocks[1].ff.gate_up.weight
    assert torch.equal(gu[:224], src.read(p + "mlp.gate_proj.weight")) and torch.equal(gu[224:], src.read(p + "mlp.up_proj.weight"))


def test_random_weights_mode(tmp_path):
    cfg, _ = model_for("C")
    a = write_random_model(cfg, tmp_path / "a", seed=3)
    b = write_random_model(cfg, tmp_path / "b", seed=3)
    c = write_random_model(cfg, tmp_path / "c", seed=4)
    sa, sb, sc = SafetensorsDir(a), SafetensorsDir(b), SafetensorsDir(c)
    assert json.loads((a / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    assert Qwen3Config.from_dict(json.loads((a / "config.json").read_text())) == cfg
    for n in sa.names():
        assert torch.equal(sa.read(n), sb.read(n)) and sa.info(n).dtype_name == "BF16"
        assert not torch.equal(sa.read(n), sc.read(n))
    w = sa.read("model.layers.0.mlp.gate_proj.weight").float()
    g = sa.read("model.layers.0.input_layernorm.weight").float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    assert abs(float(g.mean()) - 1.0) < 0.05 and 0.05 < float(g.std()) < 0.15
