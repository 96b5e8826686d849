"""The C++ driver that mirrors the reference's main() (cuSpAMM.cu:395-560) on top of the C ABI:
run it as a program and check what it prints against the checker on the same generated inputs."""
import os
import re
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
MAIN = os.path.join(HERE, "..", "cuspamm_amd", "spamm_main")


def _run(args):
    if not os.path.exists(MAIN):
        pytest.fail("cuspamm_amd/spamm_main is missing: build it with `python -m cuspamm_amd.build`")
    proc = subprocess.run([MAIN] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=120)
    assert proc.returncode == 0, proc.stdout
    return proc.stdout


@pytest.mark.parametrize("gen,c,v,tile,tau", [("exp", 1.0, 0.9, 32, 1e-2), ("alg", 0.1, 0.1, 64, 5.5)])
def test_reference_generators_through_the_driver(orc, gen, c, v, tile, tau):
    n = 1024
    out = _run(["--M", n, "--K", n, "--N", n, "--tile", tile, "--gen", gen, "--c", c, "--v", v, "--tau", tau,
                "--testtime", 4, "--warmup", 1, "--check"])
    assert "input parameters: M=1024 K=1024 N=1024" in out            # the reference's first line (cuSpAMM.cu:396)
    t = float(re.search(r"SpAMM time=([0-9.eE+-]+)s", out).group(1))   # and its last (cuSpAMM.cu:554)
    assert 0.0 < t < 1.0
    kept, total = map(int, re.search(r"valid products=(\d+) of (\d+)", out).groups())
    tab = orc.decay_table("ref_" + gen, n, c=c, v=v)
    A = orc.fill_decay(n, n, tab, 0, random=False)
    ref = orc.spamm(A, A, tile, tau)
    assert total == (n // tile) ** 3
    assert 0 < ref["kept"] < total
    # the driver builds its table with libm, the checker with numpy: allow a product or two at the threshold
    assert abs(kept - ref["kept"]) <= max(2, ref["kept"] // 1000)
    err, dense, cn, bound = map(float, re.search(
        r"\|C_dense-C\|_F=(\S+) \|C_dense\|_F=(\S+) \|C\|_F=(\S+) bound=(\S+)", out).groups())
    assert dense > 0 and err <= bound * (1 + 1e-4) + 1e-5 * dense
    assert abs(cn - np.sqrt(float((ref["C"].astype(np.float64) ** 2).sum()))) <= 1e-3 * cn


def test_driver_pads_and_tunes(orc):
    # dimensions that are not tile multiples are padded up (main.h:54-56); --ratio picks tau on the device
    out = _run(["--M", 1000, "--K", 900, "--N", 1100, "--tile", 64, "--gen", "exp", "--c", 1.0, "--v", 0.99,
                "--ratio", 0.3, "--testtime", 3, "--warmup", 0, "--prune"])
    assert "input parameters: M=1024 K=960 N=1152" in out
    ach = float(re.search(r"valid ratio=([0-9.]+)", out).group(1))
    kept, total = map(int, re.search(r"valid products=(\d+) of (\d+)", out).groups())
    assert total == 16 * 15 * 18 and abs(ach - 0.3) < 0.02 and abs(kept / total - ach) < 1e-6


def test_driver_defaults_are_the_reference_experiment_with_fp16_operands(orc):
    # no options: 2048^3, tile 32, getDecayMatrixAlg(0.1, 0.1), Norm = 1.548969 (para.h:1-14, cuSpAMM.cu:428-431);
    # --half: the operands are fp16 before the timed multiplies, as USINGHALF 1 has them
    plain, half = _run(["--check"]), _run(["--half", "--check"])
    for out in (plain, half):
        assert "input parameters: M=2048 K=2048 N=2048 Norm=1.548969" in out
    pick = lambda out: (re.search(r"valid products=(\d+) of (\d+)", out).groups(),
                        re.search(r"\|C_dense-C\|_F=(\S+) \|C_dense\|_F=(\S+) \|C\|_F=(\S+) bound=(\S+)", out).groups())
    assert pick(plain) == pick(half)            # rounding to fp16 on the host or on the device: the same operands
    kept, total = map(int, pick(half)[0])
    tab = orc.decay_table("ref_alg", 2048, c=0.1, v=0.1)
    A = orc.fill_decay(2048, 2048, tab, 0, random=False)
    ref = orc.spamm(A, A, 32, 1.548969)
    assert total == 64 ** 3 and abs(kept - ref["kept"]) <= max(2, ref["kept"] // 1000)
    proc = subprocess.run([MAIN, "--half", "--noalloc"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert proc.returncode == 2 and "--half" in proc.stdout


def test_driver_rejects_bad_arguments():
    proc = subprocess.run([MAIN, "--tile", "48"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert proc.returncode == 2 and "tile must be" in proc.stdout


def test_driver_in_the_fixed_workspace():
    # --noalloc: the timed multiplies go through spamm_multiply_noalloc; same printed counts and norms
    args = ["--M", 1024, "--K", 768, "--N", 1280, "--tile", 64, "--gen", "exp", "--c", 1.0, "--v", 0.98, "--tau", 0.05,
            "--testtime", 3, "--warmup", 0, "--check"]
    plain, fixed = _run(args), _run(args + ["--noalloc"])
    pick = lambda out: (re.search(r"valid products=(\d+) of (\d+)", out).groups(),
                        re.search(r"\|C_dense-C\|_F=(\S+) \|C_dense\|_F=(\S+) \|C\|_F=(\S+) bound=(\S+)", out).groups())
    assert pick(plain) == pick(fixed)
    kept, total = map(int, pick(fixed)[0])
    assert 0 < kept < total
    # a problem beyond the fixed workspace is refused with the library's message
    proc = subprocess.run([MAIN, "--M", "8192", "--K", "8192", "--N", "8192", "--tile", "64", "--tau", "1", "--testtime", "2",
                           "--warmup", "0", "--noalloc"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode != 0 and "fixed workspace" in proc.stdout, proc.stdout
