"""The engine at the layer sizes of Qwen2-7B (28 heads in 4 groups, head size 128,
width 3584, inner width 18944) with two layers and a small vocabulary, so that the
products' long sums and the tiles' edges at the real sizes are compared with the
plain implementation too, under the four schedules, in 32-bit and in bfloat16."""
import pytest
import torch

import helpers
import schedules

pytestmark = pytest.mark.gpu

SHAPE_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "head_dim": 128, "intermediate_size": 18944, "vocab_size": 1000, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
    "max_position_embeddings": 4096,
}
LENGTHS = [100, 70, 40, 5]
TOL = {"float32": 1e-4, "bfloat16": 4e-2}
MEAN_TOL = {"float32": 4e-6, "bfloat16": 6e-3}          # the mean deviation; observed 1.2e-6 and 1.9e-3


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    d = helpers.make_model(tmp_path_factory.mktemp("m7b"), SHAPE_7B, 21, torch.bfloat16)
    reqs = helpers.random_requests(SHAPE_7B["vocab_size"], LENGTHS, 22)
    return d, reqs, helpers.plain_logits(d, reqs)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_schedules_at_the_7b_layer_sizes(model, dt):
    from litinfer_amd.engine import Engine
    d, reqs, ref = model
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        eng = Engine.from_dir(d, dtype=dt, device="cuda:0", page_size=16, max_seqs=4, page_order_seed=5,
                              max_tokens=schedules.max_live_tokens(reqs, steps, 16 if kind == "mixed" else 64))
        out = schedules.run(eng, reqs, steps)
        worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
        mean = max(schedules.mean_err(out[r], ref[r]) for r in reqs)
        print(f"[observed] 7B sizes {dt} {kind}: largest {worst:.3e}, mean {mean:.3e}")
        assert worst < TOL[dt], f"{dt} {kind}: {worst}"
        assert mean < MEAN_TOL[dt], f"{dt} {kind}: mean deviation {mean}"
        del eng
        torch.cuda.empty_cache()
