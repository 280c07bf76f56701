"""The layer sizes of Gemma 2 2B, 9B and 27B (width, heads, head size, feed-forward width as in the reference's
configs, simply/config_lib.py:852-949) with two layers, a cut-down vocabulary and random weights: the
bfloat16 kernels at the sizes they are built for, and the float32 path, against the plain implementation."""
import pytest
import torch

import bounds
import plain_gemma2 as plain
import tiny
from simply_amd.config import EngineConfig, config_from_dict
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.loading import load_model
from simply_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

SHAPES = {
    "2b": dict(hidden_size=2304, num_attention_heads=8, num_key_value_heads=4, head_dim=256, intermediate_size=9216,
               query_pre_attn_scalar=256),
    "9b": dict(hidden_size=3584, num_attention_heads=16, num_key_value_heads=8, head_dim=256, intermediate_size=14336,
               query_pre_attn_scalar=256),
    "27b": dict(hidden_size=4608, num_attention_heads=32, num_key_value_heads=16, head_dim=128, intermediate_size=36864,
                query_pre_attn_scalar=144),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["2b", "9b", "27b"])
def test_real_layer_shapes(tmp_path, gpu_lib, shape, dtype):
    d = dict(architectures=["Gemma2ForCausalLM"], num_hidden_layers=2, vocab_size=2000, rms_norm_eps=1e-6,
             rope_theta=10000.0, sliding_window=48, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
             max_position_embeddings=8192, initializer_range=0.02, **SHAPES[shape])
    folder = write_random_model(config_from_dict(d), str(tmp_path / shape), 5, torch.bfloat16, norm_std=0.1)
    w, cfg = plain.load(folder)
    tokens = tiny.random_tokens(100, 2000, 11)
    ref = bounds.reference(w, cfg, tokens, dtype)
    ecfg = EngineConfig(activation_dtype=dtype, page_size=16, batch_size=2, max_seq_len=128, max_num_issue_tokens=128,
                        total_num_pages=16, device="cuda:0", use_graphs=True, poison_freed_pages=True)
    model, _ = load_model(folder, ecfg.dtype, "cuda:0")
    ex = Executor(model, ecfg)
    for cuts in ([100], [60, 5, 3] + [1] * 32):
        ex.add_request("r")
        out, i = [], 0
        for c in cuts:
            out.append(ex.step([StepEntry("r", tokens[i:i + c], list(range(c)))]).cpu())
            i += c
        ex.finish_request("r")
        got = torch.cat(out).double()
        if dtype == "float32":
            # sums over up to 36864 terms in 32-bit: 5e-5 of the largest logit
            assert torch.isfinite(got).all()
            assert (got - ref.want).abs().max().item() / ref.scale <= 5e-5, cuts
        else:
            ref.check(got, what=cuts)


def test_long_portions(tmp_path, gpu_lib):
    """Portions of several hundred tokens at the 2B layer sizes: the kernels for many rows (the wide
    product, the residual/norm and rotary kernels with a wave per row and a block per token, attention with
    64 query rows per workgroup over a history and a window), against the plain implementation."""
    d = dict(architectures=["Gemma2ForCausalLM"], num_hidden_layers=2, vocab_size=2000, rms_norm_eps=1e-6,
             rope_theta=10000.0, sliding_window=200, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
             max_position_embeddings=8192, initializer_range=0.02, **SHAPES["2b"])
    folder = write_random_model(config_from_dict(d), str(tmp_path / "m"), 6, torch.bfloat16, norm_std=0.1)
    w, cfg = plain.load(folder)
    tokens = tiny.random_tokens(700, 2000, 12)
    ref = bounds.reference(w, cfg, tokens, "bfloat16")
    ecfg = EngineConfig(activation_dtype="bfloat16", page_size=16, batch_size=2, max_seq_len=704, max_num_issue_tokens=704,
                        total_num_pages=48, device="cuda:0", use_graphs=False, poison_freed_pages=True)
    model, _ = load_model(folder, ecfg.dtype, "cuda:0")
    ex = Executor(model, ecfg)
    for cuts in ([700], [600, 98, 2]):
        ex.add_request("r")
        out, i = [], 0
        for c in cuts:
            out.append(ex.step([StepEntry("r", tokens[i:i + c], list(range(c)))]).cpu())
            i += c
        ex.finish_request("r")
        ref.check(torch.cat(out), what=cuts)
