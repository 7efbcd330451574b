"""Index-math check of the slot layouts of the GEMM ring loop (nmtgminor_amd/csrc/gemm_ring.hip.h).

A numpy model fills one 16 KB LDS slot exactly as the kernel's one-kilobyte global -> LDS transfers
do (lane l of transfer ii writes its 16 bytes at ii * 1024 + 16 l; the swizzle is applied to the
SOURCE address), then performs the kernel's fragment reads — ds_read_b128 for a reduction-contiguous
operand, two LDS transpose reads (ds_read_b64_tr_b16) for a row-contiguous operand — and checks that
lane l ends up with the MFMA operand the 32x32x16 instruction expects from it:
    row = tile row (l & 31) of the 32-row fragment,  k = 8 (l >> 5) .. 8 (l >> 5) + 7  of the 16-k step.

The transpose read is modelled with the lane mapping measured on the hardware with a probe kernel:
within a group of 16 lanes, lane i receives element (i & 3) of what lane 4 e + (i >> 2) read, for
e = 0..3. Also checked: fragment reads and transpose reads are LDS-bank-conflict free in the access
groups the hardware forms (64 banks of 4 bytes).
"""
import numpy as np
import pytest

SLOT_ELEMS = 128 * 64          # 16 KB of 16-bit elements
ID_K = 1 << 12                  # element id = row * ID_K + k


def swz(r):
    return (r ^ (r >> 3)) & 7


def fill_slot(kc, src, ld, rows_total, row0, j, k0):
    """src: flat memory of the operand (KC: [row][k] with pitch ld, MC: [k][row] with pitch ld)."""
    lds = np.full(SLOT_ELEMS, -1, dtype=np.int64)
    for ii in range(16):
        for l in range(64):
            if kc:
                r = 8 * ii + (l >> 3)
                c = (l & 7) ^ swz(r)
                row = min(row0 + 128 * j + r, rows_total - 1)
                off = row * ld + k0 + 8 * c
            else:
                k = 4 * ii + (l >> 4)
                c = (l & 15) ^ (4 * ((l >> 4) & 3))
                row = min(row0 + 128 * j + 8 * c, rows_total - 8)
                off = (k0 + k) * ld + row
            dst = (ii * 1024 + 16 * l) // 2
            lds[dst:dst + 8] = src[off:off + 8]
    assert (lds >= 0).all()                      # the 16 x 64 transfers tile the slot exactly
    return lds


def read_fragment(kc, lds, r0, i, kk):
    """-> [64 lanes][8] element ids, and the byte addresses each read instruction touches per lane."""
    out = np.zeros((64, 8), dtype=np.int64)
    addrs = []
    if kc:
        a = np.zeros(64, dtype=np.int64)
        for l in range(64):
            row = r0 + 32 * i + (l & 31)
            a[l] = row * 128 + (((2 * kk + (l >> 5)) ^ swz(row)) * 16)
            out[l] = lds[a[l] // 2:a[l] // 2 + 8]
        addrs.append((a, 16))
    else:
        for h in range(2):
            a = np.zeros(64, dtype=np.int64)
            raw = np.zeros((64, 4), dtype=np.int64)
            for l in range(64):
                kq = 8 * (l >> 5) + ((l >> 2) & 3)
                c = r0 // 8 + 4 * i + 2 * ((l >> 4) & 1) + ((l >> 1) & 1)
                cp = c ^ (4 * ((l >> 2) & 3))
                a[l] = kq * 256 + cp * 16 + (l & 1) * 8 + (16 * kk + 4 * h) * 256
                raw[l] = lds[a[l] // 2:a[l] // 2 + 4]
            for l in range(64):
                blk, ii = l & ~15, l & 15
                for e in range(4):
                    out[l, 4 * h + e] = raw[blk + 4 * e + (ii >> 2), ii & 3]
            addrs.append((a, 8))
    return out, addrs


def conflict_free(addr, nbytes, group):
    """Lanes are served `group` at a time; inside a group no two lanes may need the same bank."""
    for g0 in range(0, 64, group):
        banks = []
        for l in range(g0, g0 + group):
            banks += [((addr[l] + 4 * w) // 4) % 64 for w in range(nbytes // 4)]
        if len(set(banks)) != len(banks):
            return False
    return True


@pytest.mark.parametrize("kc", [True, False])
@pytest.mark.parametrize("rows_total,row0,j", [(512, 256, 0), (512, 256, 1), (200, 128, 0), (72, 0, 0), (8, 0, 0)])
def test_fragments_hold_the_mfma_operand(kc, rows_total, row0, j):
    K, k0 = 192, 64
    ld = (K if kc else rows_total) + 8          # padded leading dimension
    size = (rows_total if kc else K) * ld
    src = np.full(size, -7, dtype=np.int64)
    for row in range(rows_total):
        for k in range(K):
            src[(row * ld + k) if kc else (k * ld + row)] = row * ID_K + k
    lds = fill_slot(kc, src, ld, rows_total, row0, j, k0)
    for r0 in (0, 64):                          # wave tiles start at a multiple of their height inside the slot
        for i in range(2):
            for kk in range(4):
                frag, addrs = read_fragment(kc, lds, r0, i, kk)
                for l in range(64):
                    row = row0 + 128 * j + r0 + 32 * i + (l & 31)
                    if row >= rows_total:
                        continue                # clamped duplicates: their products are never stored
                    want = [row * ID_K + k0 + 16 * kk + 8 * (l >> 5) + e for e in range(8)]
                    assert frag[l].tolist() == want, (kc, r0, i, kk, l)
                for a, nbytes in addrs:
                    # 128-bit reads are served 16 lanes at a time, 64-bit reads 32 lanes at a time (256 B per clock)
                    assert conflict_free(a, nbytes, 16 if nbytes == 16 else 32), (kc, r0, i, kk)


def test_transfers_are_one_kilobyte_contiguous_in_lds_and_coalesced_in_memory():
    # each transfer reads whole 128-byte lines (KC: 8 rows x 128 B, MC: 4 k-rows x 256 B)
    for kc in (True, False):
        for ii in range(16):
            segs = {}
            for l in range(64):
                if kc:
                    r = 8 * ii + (l >> 3)
                    c = (l & 7) ^ swz(r)
                    segs.setdefault(r, set()).add(c)
                else:
                    k = 4 * ii + (l >> 4)
                    c = (l & 15) ^ (4 * ((l >> 4) & 3))
                    segs.setdefault(k, set()).add(c)
            assert all(v == set(range(8 if kc else 16)) for v in segs.values())
            assert len(segs) == (8 if kc else 4)
