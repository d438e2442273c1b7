"""The colour network's instruction schedule rests on one property of the matrix pipe: while a 32x32x16 MFMA occupies it
(32 cycles), the SIMD goes on issuing a few ordinary vector instructions, from the same wave and from its other wave.
The micro-benchmark that measures it is built with the library; this test runs it and checks the property, so that a
chip or compiler on which it does not hold is noticed where the schedule is decided, not as a slow frame."""
import os
import re
import subprocess

import pytest

from landmark_amd import build as B


def _rows(text):
    out = {}
    for line in text.splitlines():
        m = re.match(r"(\S+)\s+(.*?)\s+waves/SIMD (\d)\s+NM\s+(\d+) NV\s+(\d+)\s+([\d.]+) ms\s+([\d.]+) ns/trip\s+([\d.]+) ns/MFMA-slot\s+([\d.]+) shader cycles", line)
        if m:
            out[(m.group(1), m.group(2).strip(), int(m.group(3)), int(m.group(5)))] = float(m.group(9))
    return out


@pytest.mark.gpu
def test_vector_instructions_issue_under_an_mfma():
    assert os.path.exists(B.MICROBENCH_PATH), "run `python -m landmark_amd.build` first"
    text = subprocess.run([B.MICROBENCH_PATH, "2000"], check=True, capture_output=True, text=True, timeout=120).stdout
    r = _rows(text)
    mfma = r[("M", "MFMA only", 1, 0)]  # shader cycles per MFMA: 32 (8 passes of 4 cycles)
    assert 31.0 < mfma < 34.0, text
    # two fmas, or two conversion pairs (v_cvt_pk_f16_f32 + v_pk_max_f16: four instructions), per MFMA are free ...
    assert r[("MV", "MFMA + fma interleaved, same wave", 1, 2)] < 1.06 * mfma, text
    assert r[("MV", "MFMA + cvt+max interleaved, same wave", 1, 2)] < 1.06 * mfma, text
    # ... more are not: four conversion pairs per MFMA cost a third on top, sixteen fmas more than the MFMA itself
    assert r[("MV", "MFMA + cvt+max interleaved, same wave", 1, 4)] > 1.2 * mfma, text
    assert r[("MV", "MFMA + fma interleaved, same wave", 1, 16)] > 1.5 * mfma, text
    # the SIMD's oldest wave keeps the full MFMA rate whatever its other wave issues
    assert r[("M|V", "one wave MFMA, the SIMD's other wave fma", 2, 16)] < 1.06 * mfma, text
    # a chain of dependent MFMAs on one accumulator runs at the full rate
    assert r[("C", "chains 1", 1, 0)] < 1.06 * mfma, text
