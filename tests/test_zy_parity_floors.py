"""The literal tolerance as a regression guard.

Every tolerance test records, per compared tensor, the fraction of elements with
|hip - float64 oracle| <= 1e-5 + 1e-3 * |oracle| -- rtol 1e-3 / atol 1e-5 exactly as
written, no scaling (tests/parity.py).  This file runs after those tests (pytest
collects it behind them) and holds every family of this session, element-weighted, to a
floor just under what the kernels reach today, so that a change that takes a family
from 0.99999 to 0.999 fails here even though it would still be "as good as an fp32 CPU
evaluation up to k".  The fraction cannot be 1 for every family: an element near zero
of a sum with cancellation has no relative accuracy in any fp32 evaluation; the floors
of those families are the recorded values (the fp32 CPU evaluations reach 0.99999 on
grad-filter, 0.9936 ... 0.9984 on the full-size F(4x4) grad-filter samples and
0.99998 on per-activation batch-norm backward).

Families of whole deep steps (ResNet-50, where both fp32 evaluations meet the literal
bar on 10-15 % of the gradient elements only) have no floor here: they are bounded
relative to the fp32 CPU evaluation in their own tests.
"""
import pytest

import parity

pytestmark = pytest.mark.gpu

# (family prefix, floor); the first matching prefix applies
FLOORS = [
    ("conv grad-filter, winograd F(4x4), full-size layers", 0.998),
    ("conv grad-filter, winograd F(4x4)", 0.9995),
    ("conv forward", 0.9999),
    ("conv grad-data", 0.9999),
    ("conv grad-filter", 0.9999),
    ("batch norm forward, pre_activation, |mean| >> std", None),
    ("batch norm backward, pre_activation, |mean| >> std", None),
    ("batch norm", 0.9999),
    ("train step mlp", 0.9999),
    ("train step lenet5", 0.9999),
    ("train step vgg16 (reduced)", 0.9999),
    ("train step vgg16 model script (reduced)", 0.9999),
    ("vgg16 b2 layer gradients on the oracle's tensors", 0.9999),
]


def _floor_of(family):
    for prefix, floor in FLOORS:
        if family.startswith(prefix):
            return floor
    return None


def test_literal_tolerance_fraction_of_every_family_recorded_in_this_session():
    families = {}
    for r in parity.REPORT:
        f = families.setdefault(r["family"], [0.0, 0])
        f[0] += r["literal"] * r["elements"]
        f[1] += r["elements"]
    if not families:
        pytest.skip("no tolerance test ran in this session")
    checked, failures = 0, []
    for family, (met, elements) in sorted(families.items()):
        floor = _floor_of(family)
        if floor is None or elements == 0:
            continue
        checked += 1
        fraction = met / elements
        if fraction < floor:
            failures.append("%s: %.6f of %d elements meet rtol 1e-3 / atol 1e-5, floor %.4f" % (
                family, fraction, elements, floor))
    assert not failures, "; ".join(failures)
    print("%d families at or above their floors" % checked)
