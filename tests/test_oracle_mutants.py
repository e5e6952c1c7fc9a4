"""Shows that the pins in test_oracle_pins.py bite: copies of oracle/zk_oracle.c with ONE term perturbed each (the
plausible mistakes: a dropped rounding term, a negation on the other side of a shift, truncation for floor, a rounding
constant of the wrong kind, a missing clip) are compiled and the pin suite is run against each; it must fail on every one
of them and pass on the untouched copy.  CPU only; the perturbed libraries live in a temporary directory and are loaded by
nothing else.

Mutants that NO input can tell from the original are left out on purpose and listed here so that nobody adds them:
  * softmax q19 clip `d > 64<<19` against `>=` (inference/int64_gemm.cu:706), q21 `d < -(64<<21)` against `<=` (:627):
    at the boundary itself k = 92 >= 64 already gives w = 0;
  * the GEMM's `sum >> c` as a logical shift (:74): for c <= 63 bits [c, c+64) of the 128-bit sum are the same.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "oracle", "zk_oracle.c")
CFLAGS = ["-O2", "-fPIC", "-fopenmp", "-fwrapv", "-std=gnu11", "-shared"]          # oracle/Makefile's

# (name, reference line the term restates, text in zk_oracle.c, replacement, occurrence to replace: None = the only one)
MUTANTS = [
    ("softmax_q21_exponent_not_rounded", "int64_gemm.cu:634",
     "(uint64_t)d * 3025551ULL + (1ULL << 20)", "(uint64_t)d * 3025551ULL", None),
    ("softmax_q21_quotient_not_rounded", "int64_gemm.cu:657",
     "(uint64_t)num + (uint64_t)(s / 2)", "(uint64_t)num", None),
    ("softmax_q21_without_clip", "int64_gemm.cu:627",
     "if (d < -((int64_t)64 << 21)) wi = 0;", "if (0) wi = 0;", None),
    ("softmax_q19_without_clip", "int64_gemm.cu:706",
     "if (d > ((uint64_t)64 << 19)) wi = 0;", "if (0) wi = 0;", None),
    ("softmax_q19_coarser_table_index", "int64_gemm.cu:720",
     "lut[f >> 11]", "lut[(f >> 12) << 1]", None),
    ("softmax_q19_quotient_rounded", "int64_gemm.cu:740",
     "c[i] = s ? tdiv64(num, s) : 0;", "c[i] = s ? tdiv64(num + s / 2, s) : 0;", None),
    ("act_q25_negates_before_the_shift", "int64_gemm.cu:804",
     "-(int64_t)(uint64_t)(((i128)r * (i128)48408813) >> 25)",
     "(int64_t)(uint64_t)(((i128)(-r) * (i128)48408813) >> 25)", None),
    ("act_q23_negates_after_the_shift", "int64_gemm.cu:932",
     "(int64_t)(uint64_t)(((i128)(-r) * (i128)12102203) >> 23)",
     "-(int64_t)(uint64_t)(((i128)r * (i128)12102203) >> 23)", None),
    ("sigmoid_saturates_to_one_above_the_limit", "int64_gemm.cu:986-991",
     "if (r >= LIM) { C[i] = r; continue; }", "if (r >= LIM) { C[i] = mode ? LIM / 64 : r; continue; }", 0),
    ("einsum_bshd_hdc_bshc_rounds_by_half_an_ulp", "int64_gemm.cu:401",
     "1, B * S, C, D, 1, 1, (int)rescale, rescale / 2);",
     "1, B * S, C, D, 1, 1, (int)rescale, rescale ? (int64_t)1 << (rescale - 1) : 0);", None),
    ("einsum_bshc_btc_bsht_rounds_by_half_an_ulp", "int64_gemm.cu:442",
     "Bsz, S * H, T, Cdim, 1, 1, (int)rescale, rescale / 2);",
     "Bsz, S * H, T, Cdim, 1, 1, (int)rescale, rescale ? (int64_t)1 << (rescale - 1) : 0);", None),
    ("einsum_bsht_btc_bshc_rounds_by_half_an_ulp", "int64_gemm.cu:483",
     "Bsz, S * H, Cdim, T, 1, 1, (int)rescale, rescale / 2);",
     "Bsz, S * H, Cdim, T, 1, 1, (int)rescale, rescale ? (int64_t)1 << (rescale - 1) : 0);", None),
    ("einsum_bshd_hdc_bshc_without_rounding_term", "int64_gemm.cu:401",
     "1, B * S, C, D, 1, 1, (int)rescale, rescale / 2);", "1, B * S, C, D, 1, 1, (int)rescale, 0);", None),
    ("einsum_bshc_btc_bsht_without_rounding_term", "int64_gemm.cu:442",
     "Bsz, S * H, T, Cdim, 1, 1, (int)rescale, rescale / 2);", "Bsz, S * H, T, Cdim, 1, 1, (int)rescale, 0);", None),
    ("einsum_bsht_btc_bshc_without_rounding_term", "int64_gemm.cu:483",
     "Bsz, S * H, Cdim, T, 1, 1, (int)rescale, rescale / 2);", "Bsz, S * H, Cdim, T, 1, 1, (int)rescale, 0);", None),
    ("einsum_bshc_hdc_bshd_gets_a_rounding_term", "int64_gemm.cu:525",
     "1, Bsz * S, D, Cdim, 1, 1, (int)rescale, 0);", "1, Bsz * S, D, Cdim, 1, 1, (int)rescale, rescale / 2);", None),
    ("einsum_bshc_hdc_bshd_reads_weights_transposed", "int64_gemm.cu:531",
     "W + (long)h * D * Cdim, 1, Cdim, 1, 0,", "W + (long)h * D * Cdim, 1, 1, D, 0,", None),
    ("rms_norm_truncates_instead_of_floor", "int64_gemm.cu:318-321",
     "    if (rr < 0) qq -= 1;\n", "", None),
    ("rms_statistic_without_eps", "kernel.py:487",
     "u192_add128(&acc, (u128)(i128)eps);", "(void)eps;", None),
    ("gemm_operand_divisors_floor", "int64_gemm.cu:69",
     "    return a / b;\n", "    { int64_t q = a / b; if ((a % b != 0) && ((a < 0) != (b < 0))) q -= 1; return q; }\n", None),
    ("gemm_remainder_keeps_one_bit_more", "int64_gemm.cu:65",
     "(lo & ((1ULL << shift) - 1))", "(lo & ((2ULL << shift) - 1))", None),
    ("rope_products_truncate_toward_zero", "int64_gemm.cu:257-260",
     "(((i128)a * (i128)b) >> 42)", "(((i128)a * (i128)b) / ((i128)1 << 42))", None),
    ("rope_imaginary_part_subtracts", "int64_gemm.cu:263",
     "(uint64_t)mul_q42(a0, b1) + (uint64_t)mul_q42(a1, b0)", "(uint64_t)mul_q42(a0, b1) - (uint64_t)mul_q42(a1, b0)", None),
]


def _replace(text, old, new, which):
    n = text.count(old)
    if which is None:
        assert n == 1, "%r occurs %d times in zk_oracle.c: the mutant list is out of date" % (old, n)
        return text.replace(old, new)
    parts = text.split(old)
    assert n > which
    return old.join(parts[: which + 1]) + new + old.join(parts[which + 1:])


def _build(tmp, name, text):
    c = os.path.join(tmp, name + ".c")
    so = os.path.join(tmp, "lib" + name + ".so")
    with open(c, "w") as f:
        f.write(text)
    subprocess.check_call(["gcc"] + CFLAGS + ["-o", so, c, "-lm"])
    return so


def _pins(so):
    env = dict(os.environ, ZK_ORACLE_LIB=so, OMP_NUM_THREADS="2")
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_oracle_pins.py"), "-x", "-q",
                        "-p", "no:cacheprovider"], env=env, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True)
    return r.returncode, r.stdout


@pytest.fixture(scope="module")
def outcomes(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("oracle_mutants"))
    with open(SRC) as f:
        text = f.read()
    libs = {"untouched": _build(tmp, "untouched", text)}
    for name, _, old, new, which in MUTANTS:
        libs[name] = _build(tmp, name, _replace(text, old, new, which))
    with ThreadPoolExecutor(4) as pool:
        return dict(zip(libs, pool.map(_pins, libs.values())))


def test_pin_suite_passes_on_an_untouched_copy(outcomes):
    rc, out = outcomes["untouched"]
    assert rc == 0, out[-2000:]


@pytest.mark.parametrize("name,line", [(m[0], m[1]) for m in MUTANTS])
def test_pin_suite_fails_on_the_mutant(outcomes, name, line):
    rc, out = outcomes[name]
    assert rc == 1 and " failed" in out, "the pins do not notice %s (%s):\n%s" % (name, line, out[-1500:])
