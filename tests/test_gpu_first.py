"""First end-to-end check on the GPU: whole prompts, float32 and bfloat16, all tiny sizes."""

import numpy as np
import pytest
import torch

import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_logits(tmp_path, name, dtype):
    from mini_infer_amd.engine import ModelRunner, StepEntry

    cfg, block = tiny.CONFIGS[name]
    weights = tiny.make_weights(cfg, seed=ord(name))
    folder = tiny.write_model_dir(tmp_path / name, cfg, weights)
    tokens = tiny.random_tokens(cfg, 75, seed=7)
    expected = ru.oracle(cfg, weights, tokens)

    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=64, block_size=block)
    got = runner.step([StepEntry("r", tokens, list(range(len(tokens))))]).cpu().numpy()
    err = np.abs(got - expected.exact).max()
    print(f"{name} {dtype}: max |logit| {np.abs(expected.exact).max():.3f}, max err {err:.3e}, "
          f"bfloat16 storage alone {expected.yard_max:.3e}")
    ru.assert_close(got, expected, dtype, f"{name} whole prompt")
