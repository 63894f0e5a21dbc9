"""The command line without a GPU: options under the reference's names, the random-weights command."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

from dinfer_amd import cli
from tiny_configs import CONFIGS

ROOT = Path(__file__).resolve().parent.parent


def test_engine_flags_carry_the_reference_names_and_defaults():
    """bins/dinfer/src/main.rs:30-131: names and defaults of the engine-relevant flags."""
    import argparse
    p = argparse.ArgumentParser()
    cli._engine_flags(p)
    a = p.parse_args(["--model", "m"])
    assert (a.max_model_len, a.max_num_seqs, a.max_num_batched_tokens, a.block_size) == (4096, 16, 2048, 16)
    assert a.num_blocks is None and a.gpu_memory_utilization == 0.9 and a.device == 0
    assert a.long_prefill_token_threshold == 0 and a.prefill_tokens_per_step == 0
    opt = cli._options(a)
    assert opt.decode_exempt_from_budget and opt.hip_graph
    a = p.parse_args(["--model", "m", "--no-decode-exempt", "--no-cuda-graph", "--num-blocks", "77"])
    opt = cli._options(a)
    assert not opt.decode_exempt_from_budget and not opt.hip_graph and opt.num_blocks == 77
    assert not cli._options(p.parse_args(["--model", "m", "--no-hip-graph"])).hip_graph


def test_random_weights_command(tmp_path):
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIGS["A"][0]))
    out = tmp_path / "model"
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "dinfer"), "random-weights", "--config", str(cfg), "--out",
                        str(out), "--seed", "5"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
    from dinfer_amd.config import load_config
    arch, c = load_config(out)
    assert arch.name == "Qwen3ForCausalLM" and c.hidden_size == 64


def test_generate_needs_prompts(tmp_path, capsys):
    with pytest.raises(SystemExit):
        cli.main(["generate", "--model", str(tmp_path)])
    assert "prompt" in capsys.readouterr().err
