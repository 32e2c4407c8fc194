"""A training step through ``mojo_backend`` (the checks live in training_checks.py and run in a
fresh interpreter each: a process that has registered the eager ``mojo`` device cannot run a
backward pass over HIP tensors any more, see that file)."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

CHECKS = ["gpt2_training_step_gradients_match_cpu", "training_graph_runs_the_fused_attention_forward_and_backward",
          "attention_backward_follows_the_route_the_forward_took",
          "sdpa_training_graph_runs_the_fused_forward_and_backward",
          "one_sgd_step_lowers_the_loss",
          "log_softmax_and_linear_backward_in_a_compiled_graph",
          "vocabulary_projection_backward_pads_its_gradient_once",
          "cross_entropy_in_the_graph_sends_one_pass_back_to_the_logits",
          "residual_gradient_joins_inside_the_layer_norm_backward",
          "training_graphs_are_never_replayed"]


@pytest.mark.parametrize("check", CHECKS)
def test_training(check):
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "training_checks.py")
    done = subprocess.run([sys.executable, script, check], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-4000:]
    assert f"ok {check}" in done.stdout
