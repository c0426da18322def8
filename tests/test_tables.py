"""Fixed-point tables and constants of the oracle against closed forms the reference documents."""

from __future__ import annotations

import math

import numpy as np


def test_fine_sine_and_tangent_tables(oracle):
    sine, tangent = oracle.fine_tables()
    # engine.py:318-319
    assert sine[2048] == 65536 and sine[6144] == -65536
    assert sine[0] == 0 and sine[4096] == 0
    # quarter-wave symmetry of R_InitTables (engine.py:315-317)
    assert np.array_equal(sine[2049:4096], sine[:2047][::-1])
    assert np.array_equal(np.delete(sine[4096:], 2048), -np.delete(sine[:4096], 2048))
    for index in (1, 17, 1000, 2047):
        assert sine[index] == math.trunc(math.sin(index * 2 * math.pi / 8192) * 65536)
    # finetangent[2048] is tan(0) (+0.5 truncation), antisymmetric up to rounding
    assert tangent[2048] == 0
    for index in (1, 1024, 3000, 4095):
        assert tangent[index] == math.trunc(math.tan((index - 2048) * 2 * math.pi / 8192) * 65536 + 0.5)


def test_pitch_projection_offset_known_answer(oracle):
    # tests/test_rendering.py:188-193: ten binary look-down deltas pan a 192-focal view by 33.7705078125
    _sine, tangent = oracle.fine_tables()
    pitch_bam = -(182 << 16) * 10
    index = min(max(((1 << 30) - pitch_bam) >> 19, 0), 4095)
    offset = ((int(tangent[index]) * round(192.0 * 65536)) >> 16) / 65536
    assert offset == 33.7705078125
