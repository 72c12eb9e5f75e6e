"""All 36 layers of the Qwen3-8B shape: the bfloat16 engine against the float32 engine.

Both engines are tied to the plain implementation at two layers of these widths
(test_gpu_engine_full_width.py); what depth adds is compared here between the two of them, on the same
bfloat16-rounded weights, as the reference compares its fp16 path with its fp32 path on fp16-rounded weights
(crates/cuda/tests/parity.rs:22-27 for the metric, :42-45 for the calibrate-once-then-freeze bound):
finiteness first, then the row-max-normalised drift of the logits against ``helpers.DEPTH_TOL``."""
import pytest
import torch

from helpers import DEPTH_TOL, random_tokens, rel_err
from reinfer_amd import kernels
from reinfer_amd.config import config_from_dict
from reinfer_amd.engine import ModelRunner, StepEntry
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

RAW_8B = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 36, "hidden_size": 4096,
          "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
          "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
          "max_position_embeddings": 4096}


def test_bfloat16_against_float32_at_full_depth():
    """A 2,048-token prompt and seven shorter ones, then 32 decode steps of all eight together (the captured
    step of the bench), the same given tokens through both engines."""
    assert kernels.current().name == "hip-gfx950"
    cfg = config_from_dict(RAW_8B)
    dev = torch.device("cuda:0")
    weights = random_tensors(declare_params(cfg.to_spec()), 7, torch.bfloat16, dev)
    V = RAW_8B["vocab_size"]
    lens = [2048, 97, 160, 333, 512, 650, 41, 700]
    steps = 32
    seqs = {f"r{i}": random_tokens(n + steps, V, 80 + i) for i, n in enumerate(lens)}
    logits = {}
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_config(cfg, dtype=dtype, device="cuda:0", weights=weights,
                                         max_tokens=8 * 2112, max_seqs=8)
        rows = []
        for (r, s), n in zip(seqs.items(), lens):
            runner.add_request(r)
            # a prompt's first, middle and last row
            rows.append(runner.step([StepEntry(r, s[:n], [0, n // 2, n - 1])]).float().cpu())
        for k in range(steps):
            entries = [StepEntry(r, [s[n + k]], [0]) for (r, s), n in zip(seqs.items(), lens)]
            rows.append(runner.step(entries).float().cpu())
        if dtype == "bfloat16":
            assert runner.graphs is not None and runner.graphs.replays == steps
        for r in seqs:
            runner.free_request(r)
        runner.manager.check()
        logits[dtype] = rows
        del runner
        torch.cuda.empty_cache()
    worst = 0.0
    for i, (got, ref) in enumerate(zip(logits["bfloat16"], logits["float32"])):
        assert torch.isfinite(ref).all(), ("float32", i)
        assert torch.isfinite(got).all(), ("bfloat16", i)
        worst = max(worst, rel_err(got, ref))
    print(f"drift of the bfloat16 engine at 36 layers: {worst:.4f} (bound {DEPTH_TOL})")
    assert worst < DEPTH_TOL, worst
    # and it is a drift, not a constant: the two engines are different computations
    assert worst > 1e-4
