"""The world-size-1 training step (the reference's train.py loop) on a cut-down model: 2 of the 16 layers,
1024 tokens, 4 steps.  The loss of step 0 is that of a random model (about ln(vocabulary)), every step is
finite, and the weights move."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["odysseus", "tpsp"])
def test_training_steps_run(mode, dev, capsys):
    pytest.importorskip("transformers")
    from odysseus_transformer_amd import train
    from odysseus_transformer_amd.utils import globals as g
    print(f"training loop, mode {mode}", flush=True)
    args = train.parse_args(["--use_cfg_init_model", "--parallel_mode", mode, "--num-hidden-layers", "2",
                             "--seq-length", "1024", "--max-train-steps", "4", "--learning-rate", "1e-3"])
    try:
        out = train.main(args)
    finally:
        g._destroy_global_memory_buffer()
    assert out["timed_steps"] == 1 and out["layers"] == 2
    assert all(math.isfinite(l) for l in out["losses"])
    assert abs(out["losses"][0] - math.log(32000)) < 1.5
    text = capsys.readouterr().out
    assert f"{mode} 1K 1 Time taken:" in text and "CUDA memory allocated/reserved" in text
