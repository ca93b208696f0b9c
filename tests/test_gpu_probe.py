"""Checks on the hardware every lane-level assumption the kernels (and the CPU lane emulator)
rely on: MFMA operand/accumulator layouts, DPP source-lane rules, lane swaps, ballot."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_lane_primitives_match_documented_layouts():
    import tcu_scope_amd as tcu

    tcu.init(0)
    raw = tcu.lane_probe().cpu().numpy().view(np.uint32).reshape(-1, 64)
    f = raw.view(np.float32)
    lane = np.arange(64)
    n, g = lane % 16, lane // 16
    # mfma 16x16x32: D[4g+i][n] = (m+1)(n+1) for A[m][0] = m+1, B[0][n] = n+1
    for i in range(4):
        assert np.array_equal(f[0 + i], (4 * g + i + 1) * (n + 1)), f"mfma16 accumulator register {i}"
    # one-hot A[3][17] * B[17][5] lands in D[3][5] only: lane (n=5, g=0), register 3
    want = np.zeros((4, 64), np.float32)
    want[3, 5] = 1.0
    assert np.array_equal(f[4:8], want), "mfma16 k-block / row / column placement"
    # mfma 32x32x16: reg i of lane l = D[8*(i/4) + 4*(l/32) + i%4][l%32]
    for i in range(16):
        m = 8 * (i // 4) + 4 * (lane // 32) + i % 4
        assert np.array_equal(f[8 + i], (m + 1) * (lane % 32 + 1)), f"mfma32 accumulator register {i}"
    assert np.array_equal(f[24], lane ^ 1)
    assert np.array_equal(f[25], lane ^ 2)
    assert np.array_equal(f[26], (lane & ~7) | (7 - (lane & 7)))
    assert np.array_equal(f[27], (lane & ~15) | (15 - (lane & 15)))
    assert np.array_equal(f[28], np.where(n >= 1, lane, 0))          # row_shr:1 of lane+1, zero fill
    assert np.array_equal(f[29], np.where(n >= 3, lane - 2, 0))      # row_shr:3
    assert np.array_equal(f[30], lane)                               # wave_shr:1 of lane+1, lane 0 -> 0
    assert np.array_equal(f[31], np.where(g % 2 == 1, 16 * g, -1))   # row_bcast15 into rows 1,3: lane 16g-1, +1
    assert np.array_equal(f[32], np.where(g >= 2, 32, -1))           # row_bcast31 into rows 2,3
    a16 = np.where(g % 2 == 1, 100 + lane - 16, lane)
    b16 = np.where(g % 2 == 0, lane + 16, 100 + lane)
    assert np.array_equal(raw[33], a16) and np.array_equal(raw[34], b16), "permlane16_swap"
    a32 = np.where(lane >= 32, 100 + lane - 32, lane)
    b32 = np.where(lane < 32, lane + 32, 100 + lane)
    assert np.array_equal(raw[35], a32) and np.array_equal(raw[36], b32), "permlane32_swap"
    bal = sum(1 << int(l) for l in lane if l % 3 == 0)
    assert np.all(raw[37] == (bal & 0xFFFFFFFF)) and np.all(raw[38] == (bal >> 32))
    assert np.all(raw[39] == 74)
