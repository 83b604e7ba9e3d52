"""Runs the C++ harness (tests/cpp/qmm_harness.cpp): forward_qmm / backward_qmm through the C++20
shim that mirrors the reference's kernels.h, checked against the CPU oracle inside the harness."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "build", "qmm_harness")


@pytest.mark.parametrize("args", [("1024", "896", "1152", "0"), ("2048", "896", "896", "1"), ("512", "4864", "896", "0"),
                                  ("4096", "1536", "1792", "0"), ("1024", "896", "1152", "0", "1"),
                                  ("2048", "1152", "896", "1", "1"),
                                  # bf16 weight gradient; then layers with operands read in their stored layouts, "2"
                                  # where the plan expects a gain, "3" wherever the shapes are served: wgrad NT with
                                  # the copying dgrad; dgrad NN + wgrad NT; wgrad TT (OC = 9216) with the copying dgrad;
                                  # the same layer with NN + NT; wgrad TT on 224-wide tiles (C = 896); a shape no
                                  # K-major mode serves (OC = 1152); NN + NT with the quantized input reused
                                  ("1024", "1024", "1536", "0", "0", "1"), ("1024", "1024", "1536", "0", "0", "2"),
                                  ("1024", "1024", "1536", "0", "0", "3"), ("1024", "768", "9216", "0", "0", "2"),
                                  ("1024", "768", "9216", "0", "0", "3"), ("2048", "896", "768", "1", "0", "2"),
                                  ("1024", "896", "1152", "0", "1", "2"), ("512", "1536", "512", "1", "1", "3"),
                                  # fp32 weight gradients and gradient accumulation with the stored layouts ("4" / "5":
                                  # fp32 dweight; last argument: accumulate): NN + NT into fp32; NT accumulating into
                                  # bf16; TT accumulating into fp32 (OC = 9216); accumulation on the copying route
                                  ("1024", "1024", "1536", "0", "0", "5"), ("1024", "1024", "1536", "0", "0", "3", "1"),
                                  ("1024", "768", "9216", "0", "0", "4", "1"), ("1024", "1024", "1536", "0", "0", "5", "1"),
                                  ("1024", "896", "1152", "0", "0", "1", "1")])
def test_qmm_harness(args):
    assert os.path.exists(BIN), "build it with `make -C tests/cpp` (done by __graft_entry__.build())"
    r = subprocess.run([BIN, *args], capture_output=True, text=True, timeout=150)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0 and "RESULT: PASS" in r.stdout
    plan = PLANS.get(args)
    if plan is not None:
        assert "stored-layout plan: " + plan in r.stdout


# what QmmRunState::direct_layout_plan must have chosen for the stored-layout cases above
PLANS = {("1024", "1024", "1536", "0", "0", "2"): "dgrad in place 0, wgrad both in place (NT)",
         ("1024", "1024", "1536", "0", "0", "3"): "dgrad in place 1, wgrad both in place (NT)",
         ("1024", "768", "9216", "0", "0", "2"): "dgrad in place 0, wgrad gradient in place (TT)",
         ("1024", "768", "9216", "0", "0", "3"): "dgrad in place 1, wgrad both in place (NT)",
         ("2048", "896", "768", "1", "0", "2"): "dgrad in place 0, wgrad gradient in place (TT)",
         ("1024", "896", "1152", "0", "1", "2"): "dgrad in place 0, wgrad copies",
         ("512", "1536", "512", "1", "1", "3"): "dgrad in place 1, wgrad both in place (NT)",
         ("1024", "1024", "1536", "0", "0", "5"): "dgrad in place 1, wgrad both in place (NT)",
         ("1024", "1024", "1536", "0", "0", "3", "1"): "dgrad in place 1, wgrad both in place (NT)",
         ("1024", "768", "9216", "0", "0", "4", "1"): "dgrad in place 0, wgrad gradient in place (TT)",
         ("1024", "1024", "1536", "0", "0", "5", "1"): "dgrad in place 1, wgrad both in place (NT)",
         ("1024", "896", "1152", "0", "0", "1", "1"): None}
