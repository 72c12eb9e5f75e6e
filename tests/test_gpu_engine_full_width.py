"""The serving kernels at the sizes they are built for: a model with the widths of the
Qwen3-8B shape (4096 wide, 32 query heads over 8 KV heads of 128, feed-forward 12288,
vocabulary 151936) but two layers, random weights. The 32-bit path of the same engine
is the reference here (the tiny models pin that path to the plain implementation);
the bfloat16 path must agree with it under every way of cutting the work, and with
itself across cuts far more closely than bfloat16 rounding alone would demand."""
import pytest
import torch

from helpers import random_tokens, rel_err
from reinfer_amd import kernels
from reinfer_amd.config import config_from_dict
from reinfer_amd.engine import ModelRunner, StepEntry
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

RAW = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 4096,
       "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
       "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
       "max_position_embeddings": 4096}


@pytest.fixture(scope="module")
def engines():
    assert kernels.current().name == "hip-gfx950"
    cfg = config_from_dict(RAW)
    dev = torch.device("cuda:0")
    weights = random_tensors(declare_params(cfg.to_spec()), 0, torch.bfloat16, dev)
    out = {}
    for dtype in ("float32", "bfloat16"):
        out[dtype] = ModelRunner.from_config(cfg, dtype=dtype, device="cuda:0", weights=weights, max_tokens=1024,
                                             max_seqs=8)
    return out


def feed(runner, seqs, plan):
    """plan: steps of (request, n tokens); logits of every fed token per request."""
    got = {r: [] for r in seqs}
    fed = {r: 0 for r in seqs}
    for items in plan:
        entries = []
        for r, n in items:
            if not runner.has_request(r):
                runner.add_request(r)
            entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))))
        out = runner.step(entries).float().cpu()
        o = 0
        for r, n in items:
            got[r].append(out[o:o + n])
            o += n
            fed[r] += n
    for r in seqs:
        runner.free_request(r)
    return {r: torch.cat(v) for r, v in got.items()}


def test_full_width_cuts_agree(engines):
    V = RAW["vocab_size"]
    seqs = {"a": random_tokens(150, V, 1), "b": random_tokens(97, V, 2), "c": random_tokens(40, V, 3)}
    whole = [[("a", 150)], [("b", 97)], [("c", 40)]]
    ref = feed(engines["float32"], seqs, whole)
    got_whole = feed(engines["bfloat16"], seqs, whole)
    mixed = [[("a", 70), ("b", 2)], [("a", 1), ("b", 60), ("c", 17)], [("a", 65), ("b", 1), ("c", 1)],
             [("a", 1), ("b", 34), ("c", 2)]] + [[("a", 1), ("c", 1)]] * 13 + [[("c", 7)]]
    got_mixed = feed(engines["bfloat16"], seqs, mixed)
    for r in seqs:
        assert rel_err(got_whole[r], ref[r]) < 3e-2, r
        assert rel_err(got_mixed[r], ref[r]) < 3e-2, r
        # the two cuts differ by rounding only: kernels chosen by the number of rows sum in another order
        assert rel_err(got_mixed[r], got_whole[r]) < 2e-2, r
    # 32-bit: cuts agree to float rounding
    ref_mixed = feed(engines["float32"], seqs, mixed)
    for r in seqs:
        assert rel_err(ref_mixed[r], ref[r]) < 2e-5, r
