"""The quantizer kernels replace the reference's literal op sequence (src/Metis/Metis/quant.py:27-31)
by a 3-operation quotient, the hardware E2M1 converter and a few guards.  These host checks restate
both sides in C (oracle/kernel_shortcut_checks.c) and compare them: exhaustively for the bf16-per-op
mode, on adversarial block scalars for the binary32 mode.  The GPU tests then only have to show that
the device code does what the restated shortcut does."""
import os
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "oracle", "kernel_shortcut_checks")


def _run(*args):
    src = os.path.join(ROOT, "oracle", "kernel_shortcut_checks.c")
    if not os.path.exists(BIN) or os.path.getmtime(BIN) < os.path.getmtime(src):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "kernel_shortcut_checks"], check=True,
                       capture_output=True)
    env = dict(os.environ, OMP_NUM_THREADS=str(min(8, os.cpu_count() or 1)))
    out = subprocess.run([BIN, *args], capture_output=True, text=True, env=env, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "mismatches 0" in out.stdout, out.stdout
    return out.stdout


def test_block_scalar_division_by_six_is_correctly_rounded_for_every_bf16_value():
    assert "cases 32640" in _run("div6")


def test_bf16_mode_shortcut_is_exact_for_every_bf16_pair():
    text = _run("pb16")
    cases = int(text.split("cases")[1].split()[0])
    assert cases > 90_000_000                      # all (h, x) pairs times three reciprocal perturbations


def test_binary32_mode_shortcut_is_exact_outside_its_guards():
    text = _run("p32", "2000000")
    assert int(text.split("cases")[1].split()[0]) > 100_000_000
    guarded = int(text.split("guards:")[1].split()[0])
    assert 0 < guarded < 2_000_000 // 4            # the guards fire, but mostly on the adversarial families


def test_two_operation_quotient_is_exact_for_every_block_maximum_its_table_clears():
    """The row quantizer's fast path in binary32 arithmetic: a bit per bf16 block maximum says whether the quotient
    fma(x, rh, fma(x, rl, 0)) + hardware conversion reproduces the literal sequence for every bf16 element of such a
    block.  Every cleared maximum is walked here against this file's own restatement of the literal sequence
    (9e8 cases), and the table must clear all but a handful of the maxima below 2^64."""
    text = _run("table", os.path.join(ROOT, "fp4-post_amd", "csrc", "quotient_table.h"))
    assert int(text.split("cleared")[1].split(",")[0]) >= 0x5f80 - 64
    assert int(text.split("cases")[1].split()[0]) > 800_000_000


def test_binary32_values_shortcut_is_exact_outside_its_per_quotient_test():
    """Inputs that are not bf16 values (binary32 tensors, centred residuals): div3 + round-to-nearest-even
    against the literal sequence for every quotient the kernel's low-bits test does not flag."""
    text = _run("wide", "3000000")
    assert int(text.split("cases")[1].split()[0]) > 100_000_000
    assert int(text.split("literal path:")[1].split(")")[0]) > 0


def test_bf16_mode_reference_differs_from_rne_at_exactly_three_quotients():
    """Pins the three constants of the device code against the op-for-op torch restatement: over every
    bf16 q in [0, 13] compress/round (quant.py:28-31 in bf16) equals round-to-nearest-even onto the grid
    except at 5+1ulp, 7-1ulp and 10+1ulp, and it is monotone."""
    bits = torch.arange(0, 0x4200, dtype=torch.int32)
    q = (bits << 16).view(torch.float32).bfloat16()
    q = q[q.float() <= 13.0]
    qp = q - (torch.relu(q - 4) / 2 + torch.relu(q - 8) / 4)
    ref = torch.round(qp).float().clamp(max=7)
    grid = torch.tensor([0, 1, 2, 3, 4, 6, 8, 12.0])
    d = (q.float()[:, None] - grid[None, :]).abs()
    rne = d.argmin(1).float()
    tie = (d == d.min(1).values[:, None]).sum(1) > 1
    for i in torch.nonzero(tie).flatten().tolist():
        rne[i] = [c for c in torch.nonzero(d[i] == d[i].min()).flatten().tolist() if c % 2 == 0][0]
    differ = q.float()[rne != ref].tolist()
    assert differ == [5.03125, 6.96875, 10.0625]
    assert bool((ref[1:] >= ref[:-1]).all())
