"""GPU tests of the bench CLI opencnn_amd/wgrad (opencnn_amd/csrc/wgrad.hip), the re-authored
bench driver of the reference: its argument list `wgrad N C H W K C R S`
(src/openCNN_winograd.cu:246-255), the CSV prefix in_n,in_c,in_h,filt_k,filt_w, (:257,445) and
a checker line.  Each run is a child process of its own."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
WGRAD = os.path.join(ROOT, "opencnn_amd", "wgrad")


def run(*args, env=None):
    assert os.path.exists(WGRAD), "build opencnn_amd/wgrad with make -C opencnn_amd/csrc"
    e = dict(os.environ, WGRAD_ITERS="5")
    e.update(env or {})
    print("wgrad", *args, flush=True)
    return subprocess.run([WGRAD, *map(str, args)], capture_output=True, text=True, timeout=100, env=e)


def check_output(p, n, c, h, k, bound):
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.strip().splitlines()
    assert lines[0].startswith(f"{n},{c},{h},{k},3,"), lines[0]
    fields = lines[0].split(",")
    assert len(fields) == 12
    ms, ref_tflops, tflops, pct, gbs, ms_main, ms_fx = map(float, fields[5:])
    # (the three times come from separate passes of a few calls each: no order between them is asserted)
    assert ms > 0 and ms_main > 0 and ms_fx > 0 and tflops > 0 and ref_tflops > 0 and pct > 0 and gbs > 0
    m = re.search(r"\[max_error: (\S+)\]\[rel_l2: (\S+)\]\[non_finite: (\d+)\] of (\d+)", lines[-1])
    assert m, lines[-1]
    assert float(m.group(2)) <= bound and int(m.group(3)) == 0 and int(m.group(4)) == n * k * h * h


def test_reference_argument_list_on_the_plumbing_shape():
    check_output(run(32, 8, 8, 8, 64, 8, 3, 3), 32, 8, 8, 64, 1e-3)


def test_pad_stride_form_on_the_headline_layer():
    check_output(run(64, 64, 56, 56, 64, 1, 1), 64, 64, 56, 64, 1e-3)


@pytest.mark.parametrize("operands,bound", [("f16", 2e-3), ("bf16", 1.5e-2)])
def test_reduced_precision_operands(operands, bound):
    check_output(run(128, 256, 14, 14, 256, env={"WGRAD_OPERANDS": operands}), 128, 256, 14, 256, bound)


def test_a_layer_of_the_reference_sweep_with_few_tiles():
    check_output(run(32, 512, 7, 7, 512, 512, 3, 3), 32, 512, 7, 512, 1e-3)  # bench/bench.sh:18


@pytest.mark.parametrize("args", [(32, 8, 8, 8, 64, 0, 1), (32, 8, 8, 8, 64, 1, 2), (32, 8, 8, 8, 64, 8, 5, 5),
                                  (32, 8, 8, 10, 64, 8, 3, 3), (0, 8, 8, 8, 64, 8, 3, 3)])
def test_unsupported_arguments_end_with_an_error(args):
    p = run(*args)
    assert p.returncode != 0
    assert "Error occurred" in p.stderr or "wgrad:" in p.stderr
    assert "rel_l2" not in p.stdout
