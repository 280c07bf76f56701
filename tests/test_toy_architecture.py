"""A whole architecture that the package does not know (tests/toy_architecture.py: config class, block arrangement and
norm of its own) is registered from outside, written as a model folder, loaded by its config.json's name, stepped,
generated from and replayed by `bin/trace_run` in a child process, without a change to the package's files."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import toy_architecture as toy
from simply_amd import registry
from simply_amd.config import EngineConfig, config_from_dict, load_config
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.loading import load_model
from simply_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONFIG = toy.ToyConfig(width=72, depth=3, heads=6, kv_heads=2, head_size=16, inner=104, vocab=301, norm_eps=1e-4,
                       rope_base=500.0, max_positions=256)


@pytest.fixture(autouse=True)
def registered():
    toy.register()
    yield
    toy.register()  # (left registered: other test modules import nothing of it)


def folder(tmp_path, dtype=torch.float32):
    d = write_random_model(CONFIG, str(tmp_path / "toy"), seed=5, dtype=dtype, norm_std=0.3)
    from safetensors.torch import load_file

    return d, load_file(os.path.join(d, "model.safetensors"))


def tokens_of(n, seed):
    return torch.randint(0, CONFIG.vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_cut(ex, rid, tokens, cuts):
    out, i = [], 0
    ex.add_request(rid)
    for c in cuts:
        part = tokens[i:i + c]
        out.append(ex.step([StepEntry(rid, part, list(range(len(part))))]).cpu())
        i += len(part)
    ex.finish_request(rid)
    ex.cache.check()
    return torch.cat(out)


def test_the_name_in_config_json_picks_the_class(tmp_path):
    d = CONFIG.to_dict()
    assert d["architectures"] == [toy.NAME] and "hidden_size" not in d  # keys of its own
    assert config_from_dict(d) == CONFIG
    model_dir, tensors = folder(tmp_path)
    assert load_config(model_dir) == CONFIG
    assert set(tensors) == {"tok", "out", "last.gain", "last.bias"} | {
        f"blk.{i}.{n}" for i in range(3) for n in ("q", "k", "v", "o", "gate", "up", "down", "n1.gain", "n1.bias",
                                                   "n2.gain", "n2.bias")}
    toy.unregister()
    with pytest.raises(ValueError, match="Gemma2ForCausalLM"):  # unknown again: the error lists what is known
        config_from_dict(d)
    with pytest.raises(ValueError, match="keys missing"):
        toy.ToyConfig.from_dict({"architectures": [toy.NAME], "width": 8})


def test_plugins_named_in_the_environment_are_imported_once(monkeypatch, tmp_path):
    """A registry imports the modules of $SIMPLY_AMD_PLUGINS before it calls a name unknown."""
    toy.unregister()
    monkeypatch.setattr(registry, "_plugins_loaded", False)
    monkeypatch.setenv(registry.PLUGINS_ENV, "toy_architecture_plugin_probe")
    monkeypatch.syspath_prepend(str(tmp_path))
    (tmp_path / "toy_architecture_plugin_probe.py").write_text("import toy_architecture\ntoy_architecture.register()\n")
    try:
        assert registry.ARCHITECTURES.get(toy.NAME) is toy.ToyConfig
        monkeypatch.setattr(registry, "_plugins_loaded", False)
        monkeypatch.setenv(registry.PLUGINS_ENV, "no_such_module_anywhere")
        with pytest.raises(ImportError, match="no_such_module_anywhere"):
            registry.ARCHITECTURES.get("AnotherUnknownName")
    finally:
        sys.modules.pop("toy_architecture_plugin_probe", None)


def test_steps_on_the_cpu_stand_in_match_the_plain_version(tmp_path, cpu_ops):
    model_dir, tensors = folder(tmp_path)
    tokens = tokens_of(41, 1)
    want = toy.plain_logits(tensors, CONFIG, tokens)
    model, cfg = load_model(model_dir, torch.float32, "cpu")
    assert cfg == CONFIG
    ex = Executor(model, EngineConfig(activation_dtype="float32", page_size=4, batch_size=2, max_seq_len=64,
                                      max_num_issue_tokens=64, total_num_pages=40, device="cpu", use_graphs=False))
    for cuts in ([41], [9] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 9]):
        got = run_cut(ex, "r", tokens, cuts).double()
        assert (got - want).abs().max().item() <= 2e-5 * want.abs().max().item(), cuts


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_on_the_gpu_match_the_plain_version(tmp_path, gpu_lib, dtype):
    tdtype = torch.float32 if dtype == "float32" else torch.bfloat16
    model_dir, tensors = folder(tmp_path, tdtype)
    tokens = tokens_of(70, 2)
    want = toy.plain_logits(tensors, CONFIG, tokens)
    model, _ = load_model(model_dir, tdtype, "cuda:0")
    ex = Executor(model, EngineConfig(activation_dtype=dtype, page_size=16, batch_size=2, max_seq_len=128,
                                      max_num_issue_tokens=128, total_num_pages=12, device="cuda:0", use_graphs=True))
    tol = 2e-5 if dtype == "float32" else 3e-2
    whole = run_cut(ex, "r", tokens, [70]).double()
    assert (whole - want).abs().max().item() <= tol * want.abs().max().item()
    for cuts in ([38] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 9, 29]):
        got = run_cut(ex, "r", tokens, cuts).double()
        assert (got - want).abs().max().item() <= tol * want.abs().max().item(), cuts
        if dtype == "float32":
            assert (got - whole).abs().max().item() <= 1e-5 * want.abs().max().item(), cuts


@pytest.mark.gpu
def test_greedy_generation_through_the_entry_point(tmp_path, gpu_lib):
    from simply_amd import LMInterface, SamplingParams

    model_dir, tensors = folder(tmp_path)
    prompts = [tokens_of(9, 3), tokens_of(17, 4)]
    lm = LMInterface(model_dir, activation_dtype="float32", batch_size=2, max_seq_len=64, page_size=16)
    outs = lm.generate(prompts, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=12))
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for _ in range(12):
            seq.append(int(toy.plain_logits(tensors, CONFIG, seq)[-1].argmax()))
        assert list(out.output_token_ids) == seq[len(prompt):]


@pytest.mark.gpu
def test_trace_replay_in_a_child_process_with_the_plugin(tmp_path, gpu_lib):
    model_dir, tensors = folder(tmp_path)
    tokens = tokens_of(30, 6)
    want = toy.plain_logits(tensors, CONFIG, tokens)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:21], "want": [0, 20]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[21:], "want": list(range(9))}], "end": ["a"]}]
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([os.path.dirname(__file__), os.environ.get("PYTHONPATH", "")]))
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", "float32",
               "--out", str(tmp_path / "out"), "--max-tokens", "64"]
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    without = subprocess.run(command, input=text, capture_output=True, text=True, timeout=300, env=env)
    assert without.returncode != 0 and toy.NAME in without.stderr and "Gemma2ForCausalLM" in without.stderr
    env[registry.PLUGINS_ENV] = "toy_architecture"
    done = subprocess.run(command, input=text, capture_output=True, text=True, timeout=300, env=env)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1"]
    got = np.concatenate([np.fromfile(str(tmp_path / "out" / f"{i}.f32"), dtype="<f4").reshape(-1, CONFIG.vocab)
                          for i in range(2)])
    rows = [0, 20] + list(range(21, 30))
    assert np.abs(got - want[rows].numpy()).max() <= 2e-5 * float(want.abs().max())
