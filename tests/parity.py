"""Shared yardsticks of the GPU parity tests.

Three measurements are taken for every compared tensor and appended to a report
that the session writes as ``parity_report.json`` into the run's output folder (see
``write_report``; read by nobody at run time; the per-family figures quoted in the
design notes come from it):

  literal   fraction of elements with |got - ref| <= 1e-5 + 1e-3 * |ref| -- the plain
            rtol 1e-3 / atol 1e-5 bar, with no scaling of the absolute term;
  err_hip   largest |got - ref64| over the tensor (and the root-mean-square one);
  err_cpu32 the same for the float32 evaluation of the CPU oracle on the same inputs,
            i.e. for what a numpy fp32 executor would produce.

``compare`` asserts err_hip <= k * err_cpu32 (+ one rounding step of the largest
reference magnitude, so that an exactly representable result cannot make the bound
zero): the HIP result is no further from the exact answer than a plain fp32 CPU
evaluation is, up to the stated factor k.  It also asserts the literal bar relative to
that evaluation: the fraction of elements that meet it may trail the fp32 CPU
evaluation's own fraction by at most 1e-3 (+ one element).
"""
import json
import os
import zlib

import numpy as np

REPORT = []
ULP = float(np.finfo(np.float32).eps)


def stable_seed(case):
    """Seed that depends on the case's text only (Python's hash() of a str changes per process)."""
    return zlib.crc32(repr(case).encode()) & 0x7fffffff


def literal_fraction(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if got.size == 0:
        return 1.0
    return float(np.mean(np.abs(got - ref) <= 1e-5 + 1e-3 * np.abs(ref)))


def errors(got, ref):
    diff = np.asarray(got, dtype=np.float64) - np.asarray(ref, dtype=np.float64)
    if diff.size == 0:
        return 0.0, 0.0
    return float(np.abs(diff).max()), float(np.sqrt(np.mean(diff * diff)))


def compare(got, ref64, ref32, family, what, k, assert_ratio=True):
    """Record the three measurements; assert the HIP error against k x the fp32 CPU error
    in both the max and the rms norm."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    hip_max, hip_rms = errors(got, ref64)
    cpu_max, cpu_rms = errors(ref32, ref64)
    scale = float(np.abs(ref64).max()) if ref64.size else 0.0
    rec = {"family": family, "what": what, "elements": int(ref64.size), "literal": literal_fraction(got, ref64),
           "literal_cpu32": literal_fraction(ref32, ref64), "scale": scale,
           "err_hip_max": hip_max, "err_cpu32_max": cpu_max, "err_hip_rms": hip_rms, "err_cpu32_rms": cpu_rms}
    REPORT.append(rec)
    if assert_ratio:
        floor = ULP * max(scale, 1e-30)
        assert hip_max <= k * cpu_max + floor, \
            "%s: largest error %.3g exceeds %g x the fp32 CPU evaluation's %.3g" % (what, hip_max, k, cpu_max)
        assert hip_rms <= k * cpu_rms + floor, \
            "%s: rms error %.3g exceeds %g x the fp32 CPU evaluation's %.3g" % (what, hip_rms, k, cpu_rms)
        # the literal bar: no element count worth mentioning may fail it that the fp32 CPU evaluation passes
        margin = 1e-3 + 1.0 / max(1, rec["elements"])
        assert rec["literal"] >= rec["literal_cpu32"] - margin, \
            "%s: %.6f of the elements meet rtol 1e-3 / atol 1e-5, the fp32 CPU evaluation reaches %.6f" % (
                what, rec["literal"], rec["literal_cpu32"])
    return rec


def write_report(root):
    if not REPORT:
        return
    out_dir = os.environ.get("TINYFLOW_PARITY_REPORT_DIR") or os.path.join(root, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        families = {}
        for r in REPORT:
            f = families.setdefault(r["family"], {"tensors": 0, "elements": 0, "literal_elements": 0.0,
                                                  "literal_cpu32_elements": 0.0, "worst_literal": 1.0,
                                                  "worst_ratio_max": 0.0, "worst_ratio_rms": 0.0})
            f["tensors"] += 1
            f["elements"] += r["elements"]
            f["literal_elements"] += r["literal"] * r["elements"]
            f["literal_cpu32_elements"] += r["literal_cpu32"] * r["elements"]
            f["worst_literal"] = min(f["worst_literal"], r["literal"])
            if r["err_cpu32_max"] > 0:
                f["worst_ratio_max"] = max(f["worst_ratio_max"], r["err_hip_max"] / r["err_cpu32_max"])
            if r["err_cpu32_rms"] > 0:
                f["worst_ratio_rms"] = max(f["worst_ratio_rms"], r["err_hip_rms"] / r["err_cpu32_rms"])
        for f in families.values():
            n = max(1, f["elements"])
            f["literal_fraction"] = f.pop("literal_elements") / n
            f["literal_fraction_cpu32"] = f.pop("literal_cpu32_elements") / n
        with open(os.path.join(out_dir, "parity_report.json"), "w") as fh:
            json.dump({"families": families, "records": REPORT}, fh, indent=1)
    except OSError:
        pass
