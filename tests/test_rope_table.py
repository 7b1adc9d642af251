"""The llama3-scaled frequency table pinned by values worked out by hand from the rule of
cwm/fastgen/forward.py:1031-1047, for the plain implementation and for the product's part alike.

The reference holds no vector of this table, so the numbers below are the rule applied on paper:
    f_i        = theta ** -(2 i / head_dim)
    wavelength = 2 pi / f_i
    long  (wavelength > old / low):   f_i / factor
    short (wavelength < old / high):  f_i
    band between:                     s = (old / wavelength - low) / (high - low);  f_i ((1 - s) / factor + s)
Each band entry is written out with its s, so a blend with s and 1 - s exchanged, a band rule applied to
the divided value, or a border on the wrong side gives another number (the exchanged blend is asserted to differ).
"""

import math

import pytest
import torch

from cwm_amd.parts.rope import RotaryEncoding
from plain import llama3_plain as plain

# (head_dim, theta, scaling) -> {index: (value, blend s or None)}
CASES = [
    # Tiny-B's table: 2 pi / 10**-0.375 = 14.8998 lies between 32/4 and 32/1
    (
        32,
        1e6,
        {"scale_factor": 4, "old_context_len": 32, "low_freq_factor": 1, "high_freq_factor": 4},
        {
            0: (1.0, None),  # wavelength 6.28 < 8: untouched
            # f = 10**-0.375 = 0.42169650; 32 / 14.8998 = 2.147684; s = 1.147684 / 3 = 0.382561;
            # 0.617439 / 4 + 0.382561 = 0.536921; 0.42169650 * 0.536921 = 0.2264176
            1: (0.2264176, 0.382561),
            2: (0.1778279 / 4, None),  # f = 10**-0.75, wavelength 35.3 > 32: divided
            15: (10 ** -5.625 / 4, None),
        },
    ),
    # the 32B shape's table: the band is 2,048 <= wavelength <= 8,192, indices 27 to 33 of 64
    (
        128,
        1e6,
        {"scale_factor": 16, "old_context_len": 8192, "low_freq_factor": 1, "high_freq_factor": 4},
        {
            26: (10 ** (-6 * 26 / 64), None),  # wavelength 1,720.6: the last short one
            # f = 10**-2.53125 = 2.9427272e-3; wavelength 2,135.16; 8192 / 2135.16 = 3.836718;
            # s = 2.836718 / 3 = 0.945573; 0.054427 / 16 + 0.945573 = 0.948974; product 2.7925743e-3
            27: (2.7925743e-3, 0.945573),
            # f = 10**-2.8125 = 1.5399265e-3; wavelength 4,080.18; 8192 / 4080.18 = 2.007754;
            # s = 1.007754 / 3 = 0.335918; 0.664082 / 16 + 0.335918 = 0.377423; product 5.8120294e-4
            30: (5.8120294e-4, 0.335917),
            # f = 10**-3.09375 = 8.0584219e-4; wavelength 7,797.04; 8192 / 7797.04 = 1.050655;
            # s = 0.050655 / 3 = 0.016885; 0.983115 / 16 + 0.016885 = 0.078330; product 6.3121332e-5
            33: (6.3121332e-5, 0.016885),
            34: (10 ** (-6 * 34 / 64) / 16, None),  # wavelength 10,179: the first long one
            63: (10 ** (-6 * 63 / 64) / 16, None),
        },
    ),
]


def _tables(head_dim, theta, scaling):
    return {
        "plain": plain.rope_frequencies(head_dim, theta, scaling),
        "product": RotaryEncoding(head_dim, theta, scaling).host_table,
    }


@pytest.mark.parametrize("head_dim,theta,scaling,entries", CASES)
def test_llama3_table_against_values_worked_out_by_hand(head_dim, theta, scaling, entries):
    for who, table in _tables(head_dim, theta, scaling).items():
        assert table.dtype == torch.float32 and table.shape == (head_dim // 2,)
        for index, (value, blend) in entries.items():
            got = float(table[index])
            assert math.isclose(got, value, rel_tol=2e-6), f"{who}: entry {index} is {got}, by hand {value}"
            if blend is not None:
                base = theta ** (-2 * index / head_dim)
                exchanged = base * (blend / scaling["scale_factor"] + (1 - blend))
                assert not math.isclose(got, exchanged, rel_tol=1e-2), f"{who}: entry {index} blends the wrong way round"


@pytest.mark.parametrize("head_dim,theta,scaling,entries", CASES)
def test_llama3_table_of_plain_and_product_agree_everywhere(head_dim, theta, scaling, entries):
    tables = _tables(head_dim, theta, scaling)
    assert torch.equal(tables["plain"], tables["product"])
    # the band rises monotonically from the divided to the untouched frequencies
    base = plain.rope_frequencies(head_dim, theta)
    ratio = (tables["plain"] / base).double()
    assert (ratio[1:] <= ratio[:-1] + 1e-7).all() and math.isclose(float(ratio.max()), 1.0) and math.isclose(float(ratio.min()), 1 / scaling["scale_factor"], rel_tol=1e-6)


def test_table_without_scaling_is_the_power_law():
    for who, table in _tables(48, 5e5, None).items():
        want = torch.tensor([5e5 ** (-2 * i / 48) for i in range(24)], dtype=torch.float64)
        torch.testing.assert_close(table.double(), want, rtol=2e-6, atol=0)
