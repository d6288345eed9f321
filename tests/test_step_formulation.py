"""The decode step as the hand-scheduled kernels compute it (csrc/fast_tile.h), restated in plain integers and
checked against the plain-integer encoder: state kept scaled by 8 so that the table address is one AND, one table
entry per slot holding 8 * freq with the symbol in the top byte and 8 * (slot - cdf), a 24-bit multiply that
ignores that top byte, one byte taken where the new state is below 2^16 and a second where it still is.  What the
test pins are the ranges the formulation relies on, for every table shape a plane can produce."""
import numpy as np
import pytest

import pyref

L8 = (1 << 16) << 3
MASK24 = (1 << 24) - 1


def _slot_table_x8(freq, cdf):
    """build_slot_table_x8: .x = 8 * freq | symbol << 24, .y = 8 * (slot - cdf)."""
    lo, hi = np.zeros(4096, np.int64), np.zeros(4096, np.int64)
    for s in range(256):
        f, c = int(freq[s]), int(cdf[s])
        for slot in range(c, c + f):
            lo[slot] = (f << 3) | (s << 24)
            hi[slot] = (slot - c) << 3
    return lo, hi


def _decode_scaled(state, data, n, lo, hi):
    """n symbols from one stream; `data` in emission order (the decoder reads it from the end)."""
    X, pos, out = state << 3, len(data) - 1, []
    for _ in range(n):
        assert L8 <= X < (1 << 27) and X & 7 == 0                   # 2^16 <= state < 2^24, nothing in the low bits
        addr = X & 0x7FF8                                           # v_and_b32: byte address of the 8-byte entry
        e_lo, e_hi = int(lo[addr >> 3]), int(hi[addr >> 3])
        q = X >> 15                                                 # state >> 12
        assert q <= MASK24 and (e_lo & MASK24) == (e_lo & 0xFFFF)   # both factors fit the 24-bit multiplier
        X = (e_lo & MASK24) * (q & MASK24) + e_hi                   # v_mad_u32_u24
        assert X < (1 << 32)
        out.append(e_lo >> 24)
        for _ in range(2):                                          # masked byte, then the rare second one
            if X < L8:
                byte = data[pos] if pos >= 0 else 0
                pos -= 1
                X = ((X << 8) | (byte << 3)) & 0xFFFFFFFF           # v_lshl_or_b32 with the byte shifted by 3
        assert X >= L8 or pos < -1                                  # two bytes always suffice
    return out, X >> 3, pos


@pytest.mark.parametrize("kind", ["zipf", "two_symbols", "uniform", "one_rare", "bf16_exponents"])
def test_scaled_step_decodes_what_the_integer_encoder_wrote(oracle, kind):
    rng = np.random.default_rng(7)
    n = 3000
    if kind == "zipf":
        p = 1.0 / np.arange(1, 257) ** 1.3
        sym = rng.choice(256, n, p=p / p.sum())
    elif kind == "two_symbols":
        sym = rng.choice([3, 200], n, p=[0.97, 0.03])
    elif kind == "uniform":
        sym = rng.integers(0, 256, n)
    elif kind == "one_rare":                                        # frequency 1 next to frequency ~3800: two-byte steps
        sym = np.full(n, 17)
        sym[rng.choice(n, 12, replace=False)] = 99
    else:
        w = (rng.standard_normal(n) * 0.02).astype(np.float32)
        sym = (w.view(np.uint32) >> 23) & 0xFF
    sym = sym.astype(np.uint8)
    freq, cdf = oracle.get_lut(sym)
    assert int(freq.min()) >= 1 and (int(freq.max()) << 3) < (1 << 24)   # 8 * freq stays below the symbol byte
    lo, hi = _slot_table_x8(freq, cdf)
    state, data = pyref.encode_stream(sym.tolist(), freq, cdf)
    out, end, pos = _decode_scaled(state, data, n, lo, hi)
    assert out == sym.tolist()
    assert end == 1 << 16 and pos == -1                             # back at the start state, every byte consumed
