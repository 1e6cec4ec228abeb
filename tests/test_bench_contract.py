"""What the measurement program promises without a GPU: its options, and its refusal of more than one GPU."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, timeout=120)


def test_more_than_one_gpu_is_refused_with_one_line_and_status_two():
    proc = run("--gpus", "2", "--steps", "3", "--warmup", "1")
    assert proc.returncode == 2
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_options_of_the_contract_are_accepted():
    import bench
    args = bench.parse_args(["--gpus", "1", "--steps", "7", "--warmup", "2"])
    assert (args.gpus, args.steps, args.warmup, args.batch, args.context, args.prefill_tokens) == (1, 7, 2, 8, 2048, 2048)
    assert bench.PEAK_HBM_GBS == 8000.0 and bench.PEAK_FLOPS == {"bf16": 2.5e15, "fp32": 157.3e12}


def test_flops_and_bytes_of_the_headline_shape():
    """The counts that the roofline fractions are priced with: 28 layers of 100.7 M matrix weights (201.3 MB in
    bfloat16), the head once."""
    import bench
    from simple_inference_amd import preset
    from simple_inference_amd.config.model_config import LlamaConfig
    mc = LlamaConfig.from_dict(preset("llama-3.2-3b"))
    layers, head = bench.matmul_params(mc)
    assert layers == 28 * 100_663_296 and head == 128256 * 3072
    assert mc.kv_bytes_per_token(2) == 28 * 8 * 128 * 2 * 2


def test_decode_allowance_covers_the_steps_that_build_the_contexts():
    """Requests decode while the other prompts of their batch are still run in portions: they may generate one token
    for every such step on top of the measured ones, or the first of them would end before the measurement does."""
    import bench
    assert bench.decode_allowance(2048, 8, 2048) == 8 + 2
    assert bench.decode_allowance(2048, 8, 8192) == 8 * 4 + 2
    assert bench.decode_allowance(2048, 64, 2049) == 64 * 2 + 2


def test_the_bound_on_the_logits_is_the_measured_one_at_the_headline_depth():
    import bench
    assert bench.logit_bound(28) == 5.0e-2 and 1.3e-2 < bench.logit_bound(2) < 1.4e-2
