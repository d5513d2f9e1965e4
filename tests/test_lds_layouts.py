"""Bank-conflict freedom of the staging layouts of the persistent tile kernels, from the address formulas in the kernel
sources and the way this chip serves wide LDS accesses (measured with conflict counters: a 16-byte access of a wave is
served in four passes of 16 lanes - {0-3, 12-15, 20-23, 24-27}, the same + 32, {4-7, 8-11, 16-19, 28-31}, the same + 32 -
and an 8-byte access in two passes of 32 consecutive lanes; a pass is conflict-free when its lanes touch every one of the
64 four-byte banks at most once)."""
import pytest

B128_PASSES = [[*range(0, 4), *range(12, 16), *range(20, 24), *range(24, 28)], [*range(4, 8), *range(8, 12), *range(16, 20), *range(28, 32)]]
B128_PASSES = [p for q in B128_PASSES for p in (q, [l + 32 for l in q])]
B64_PASSES = [list(range(0, 32)), list(range(32, 64))]


def _banks(addr, nbytes):
    return [((addr + 4 * i) // 4) % 64 for i in range(nbytes // 4)]


def _conflict_free(passes, addr_of_lane, nbytes):
    for lanes in passes:
        seen = [b for l in lanes for b in _banks(addr_of_lane(l), nbytes)]
        if len(seen) != len(set(seen)):
            return False
    return True


@pytest.mark.parametrize("bj", range(8))
def test_gemm16_persistent_staging_writes(bj):
    # gemm16_tile256p.h, stage_rows: row r16 = lane % 16, g = lane / 16; 8 bytes at r16*256 + (((g>>1) ^ r16) ^ 2 bj)*16 + (g&1)*8
    assert _conflict_free(B64_PASSES, lambda l: (l % 16) * 256 + ((((l // 16) >> 1) ^ (l % 16)) ^ (2 * bj)) * 16 + ((l // 16) & 1) * 8, 8)


@pytest.mark.parametrize("p", range(4))
def test_gemm16_persistent_staging_reads(p):
    # drain: row 4p + lane/16, chunk lane%16 at position (lane%16 ^ lane/16) ^ 4p
    assert _conflict_free(B128_PASSES, lambda l: (l // 16) * 256 + p * 1024 + (((l % 16) ^ (l // 16)) ^ (4 * p)) * 16, 16)


@pytest.mark.parametrize("h,bj", [(h, bj) for h in range(2) for bj in range(8)])
def test_fp8_persistent_staging_writes(h, bj):
    # fp8_gemm_tile256p.h, stage_rows: row = 16 h + r16; 8 bytes at row*256 + ((2 bj + (gq>>1)) ^ (row & 15))*16 + (gq&1)*8
    def addr(l):
        r16, gq = l % 16, l // 16
        row = 16 * h + r16
        return row * 256 + ((2 * bj + (gq >> 1)) ^ (row & 15)) * 16 + (gq & 1) * 8
    assert _conflict_free(B64_PASSES, addr, 8)


@pytest.mark.parametrize("p", range(8))
def test_fp8_persistent_staging_reads(p):
    # drain: row = 4p + lane/16, chunk ch = lane%16 at position ch ^ (row & 15)
    def addr(l):
        row, ch = 4 * p + l // 16, l % 16
        return row * 256 + (ch ^ (row & 15)) * 16
    assert _conflict_free(B128_PASSES, addr, 16)


def test_the_check_sees_a_conflict():
    # rows of 256 bytes without a swizzle: the 16 lanes of a column all hit the same banks
    assert not _conflict_free(B64_PASSES, lambda l: (l % 16) * 256 + (l // 16) * 8, 8)
