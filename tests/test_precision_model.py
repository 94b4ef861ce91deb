"""The operand formats of the chunked WKV7 forward kernel (jaxrwkv_amd/csrc/wkv7_fwd.hip), checked on the CPU.

tests/precision_model.py evaluates the kernel's chunk algebra in float64 with each matrix-core operand rounded the
way the kernel rounds it.  These tests pin three facts the kernel's design rests on:

  * the model with exact operands IS the recurrence (so what the other rows measure is operand rounding only);
  * the chosen set (fp16 everywhere, bf16 pairs for the four Gram operands) keeps the proxy of the logits
    total-variation distance under 1e-3 and y within 5e-4 relative rms, on fast and on slow decays;
  * the cheaper sets (single bf16 everywhere; single-bf16 Gram operands; single-bf16 at/qt in the Gram tiles) do not,
    which is why the kernel pays for the 3-term bf16 products in the Gram tiles.

The GPU tests (tests/test_gpu_wkv7_chunked.py) hold the kernel itself to tolerances derived from these figures.
"""
import pytest

from . import precision_model as pm

SHAPE = dict(B=1, T=512, H=4)


@pytest.fixture(scope="module", params=["bench", "slow"])
def case(request):
    x = pm.make_inputs(request.param, **SHAPE)
    m, ref = pm.metrics(x, pm.EXACT)
    return x, ref, m


def test_exact_operands_reproduce_the_recurrence(case):
    _, _, m = case
    assert m["y"] < 1e-6 and m["sa"] < 1e-6
    assert m["s"] < 1e-6          # the model rounds the carried state to fp32 after every chunk, as the kernel does
    assert m["tvd_max"] < 1e-4


def test_chosen_formats_meet_the_bf16_bar(case):
    x, ref, _ = case
    m, _ = pm.metrics(x, pm.CHOSEN, ref)
    assert m["tvd_max"] < 1e-3, m
    assert m["y"] < 5e-4 and m["s"] < 5e-4 and m["sa"] < 7e-4, m


@pytest.mark.parametrize("name,override", [
    ("single bf16 everywhere", pm.ALL_BF16),
    ("Gram operands single bf16", {**pm.CHOSEN, "gk": "b1", "ga": "b1"}),
    ("at/qt single bf16 in the Gram tiles", {**pm.CHOSEN, "ga": "b1"}),
])
def test_cheaper_formats_miss_it(case, name, override):
    x, ref, _ = case
    m, _ = pm.metrics(x, override, ref)
    assert m["tvd_max"] > 1e-3 and m["y"] > 1e-3, (name, m)


def test_pairs_everywhere_is_two_orders_better_but_not_needed(case):
    x, ref, _ = case
    m, _ = pm.metrics(x, pm.ALL_SPLIT, ref)
    assert m["y"] < 3e-5 and m["tvd_max"] < 1e-3, m
