"""CPU emulation of the register-level tricks the HIP kernels rely on.

Each helper below mirrors one device routine instruction by instruction (v_perm_b32,
v_and_or_b32 with the fp16 magic numbers, the SWAR sign extension, the LDS swizzle), so an index
or selector mistake shows up here, without a GPU.  The expected values come from the oracle.
"""
import numpy as np
import pytest
import torch

from oracle import ref


def v_perm_b32(s0: int, s1: int, sel: int) -> int:
    """D.byte[i] = {s0 (bytes 4..7), s1 (bytes 0..3)}.byte[sel.byte[i]] for selector values 0..7."""
    pool = [(s1 >> (8 * i)) & 0xFF for i in range(4)] + [(s0 >> (8 * i)) & 0xFF for i in range(4)]
    out = 0
    for i in range(4):
        out |= pool[(sel >> (8 * i)) & 0xFF] << (8 * i)
    return out


def half_bits_to_float(b: int) -> float:
    return float(np.array([b], dtype=np.uint16).view(np.float16)[0])


def test_fp16_magic_numbers():
    # (x & 0x000f) | 0x6400 == 1024 + u ; (x & 0x00f0) | 0x5400 == 64 + u
    for u in range(16):
        assert half_bits_to_float(u | 0x6400) == 1024.0 + u
        assert half_bits_to_float((u << 4) | 0x5400) == 64.0 + u
        # bf16: 0x4300 | u == 128 + u
        f = np.array([(0x4300 | u) << 16], dtype=np.uint32).view(np.float32)[0]
        assert f == 128.0 + u


def expand8_f16(word: int, s: np.float16, z: np.float16, fold: bool):
    """Mirror of Expand8<half_t>::operator() in csrc/gemm_w4a16.hip: returns 8 fp16 in k order."""
    def pair(x, mask, magic):
        v = (x & mask) | magic
        return np.array([v & 0xFFFF, v >> 16], dtype=np.uint16).view(np.float16)

    b_lo = np.float16(1024.0 + float(z)) if fold else np.float16(1024.0)
    b_hi = np.float16(64.0 + float(z)) if fold else np.float16(64.0)
    v8 = word >> 8
    p = [pair(word, 0x000F000F, 0x64006400) - b_lo, pair(word, 0x00F000F0, 0x54005400) - b_hi,
         pair(v8, 0x000F000F, 0x64006400) - b_lo, pair(v8, 0x00F000F0, 0x54005400) - b_hi]
    p = [q.astype(np.float16) for q in p]
    if not fold:
        p = [(q - z).astype(np.float16) for q in p]
    p = [(q * s).astype(np.float16) for q in p]
    a = [int(q.view(np.uint16)[0]) | (int(q.view(np.uint16)[1]) << 16) for q in p]
    o = [v_perm_b32(a[1], a[0], 0x05040100), v_perm_b32(a[3], a[2], 0x05040100),
         v_perm_b32(a[1], a[0], 0x07060302), v_perm_b32(a[3], a[2], 0x07060302)]
    halves = []
    for w in o:
        halves += [w & 0xFFFF, w >> 16]
    return np.array(halves, dtype=np.uint16)


@pytest.mark.parametrize("fold,zval", [(True, 8.0), (True, 0.0), (False, 7.0), (False, 6.4140625)])
def test_expand8_f16_matches_oracle(fold, zval):
    rng = np.random.default_rng(0)
    words = rng.integers(0, 2**32, size=64, dtype=np.uint64)
    s = np.float16(0.0137)
    z = np.float16(zval)
    for w in words:
        w = int(w)
        got = expand8_f16(w, s, z, fold)
        packed = torch.tensor([[(w >> (8 * i)) & 0xFF for i in range(4)]], dtype=torch.uint8)
        want = ref.dequant_w4(packed, torch.tensor([[float(s)]], dtype=torch.float16),
                              torch.tensor([[float(z)]], dtype=torch.float16), 8, torch.float16)
        assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16)[0]), hex(w)


def test_gemv_pair_order():
    """The GEMV kernel multiplies unpack pair 4*j+i = (k0+i, k0+i+4) of word j with the activation
    pair built by load_act: check both index maps name the same elements."""
    K = 32
    for j in range(4):
        word_nibbles = list(range(8 * j, 8 * j + 8))
        # unpack: p0=(k0,k4) p1=(k1,k5) p2=(k2,k6) p3=(k3,k7)
        unpack_pairs = [(word_nibbles[i], word_nibbles[i + 4]) for i in range(4)]
        # load_act: q0=(0,1) q1=(2,3) q2=(4,5) q3=(6,7) of this group of 8
        q = [(8 * j + 2 * t, 8 * j + 2 * t + 1) for t in range(4)]
        act_pairs = [(q[0][0], q[2][0]), (q[0][1], q[2][1]), (q[1][0], q[3][0]), (q[1][1], q[3][1])]
        assert unpack_pairs == act_pairs
    assert K == 32


def transpose4x4_bytes(a, b, c, d):
    """Mirror of the 4x4 byte transpose in I8KNLoader::lstore."""
    ab_lo = v_perm_b32(b, a, 0x05010400)
    ab_hi = v_perm_b32(b, a, 0x07030602)
    cd_lo = v_perm_b32(d, c, 0x05010400)
    cd_hi = v_perm_b32(d, c, 0x07030602)
    return [v_perm_b32(cd_lo, ab_lo, 0x05040100), v_perm_b32(cd_lo, ab_lo, 0x07060302),
            v_perm_b32(cd_hi, ab_hi, 0x05040100), v_perm_b32(cd_hi, ab_hi, 0x07060302)]


def test_int8_transpose_selectors():
    rows = [0x03020100, 0x13121110, 0x23222120, 0x33323130]  # byte = 16*row + col
    t = transpose4x4_bytes(*rows)
    for j in range(4):
        assert [(t[j] >> (8 * i)) & 0xFF for i in range(4)] == [16 * i + j for i in range(4)]


def test_h16_transpose_selectors():
    # word w of row r holds columns (2w, 2w+1); element value = 256*r + col
    def word(r, w):
        return (256 * r + 2 * w) | ((256 * r + 2 * w + 1) << 16)

    for w in range(4):
        a, b, c, d = (word(r, w) for r in range(4))
        even = (v_perm_b32(b, a, 0x05040100), v_perm_b32(d, c, 0x05040100))
        odd = (v_perm_b32(b, a, 0x07060302), v_perm_b32(d, c, 0x07060302))
        for col, pair in ((2 * w, even), (2 * w + 1, odd)):
            vals = [pair[0] & 0xFFFF, pair[0] >> 16, pair[1] & 0xFFFF, pair[1] >> 16]
            assert vals == [256 * r + col for r in range(4)]


def sign4(x: int, mode: str) -> int:
    """Mirror of W4I8Loader::sign4 (four nibbles, one per byte)."""
    if mode == "unsigned":
        return x
    if mode == "twos":
        x ^= 0x08080808
    c = 0x07070707 if mode == "offset7" else 0x08080808
    return (((x | 0x80808080) - c) & 0xFFFFFFFF) ^ 0x80808080


@pytest.mark.parametrize("mode", ["unsigned", "twos", "offset8", "offset7"])
def test_swar_sign_extension(mode):
    want = {"unsigned": lambda u: u, "twos": lambda u: u - 16 if u >= 8 else u, "offset8": lambda u: u - 8,
            "offset7": lambda u: u - 7}[mode]
    rng = np.random.default_rng(1)
    for _ in range(200):
        nib = [int(v) for v in rng.integers(0, 16, size=4)]
        x = sum(n << (8 * i) for i, n in enumerate(nib))
        got = sign4(x, mode)
        out = [((got >> (8 * i)) & 0xFF) for i in range(4)]
        assert out == [want(n) & 0xFF for n in nib]


def test_w4i8_expand_order():
    # expand(): lo = nibbles k0,k2,k4,k6 ; hi = k1,k3,k5,k7 ; perm(hi, lo, 0x05010400) = k0 k1 k2 k3
    v = 0x76543210
    lo, hi = v & 0x0F0F0F0F, (v >> 4) & 0x0F0F0F0F
    d0, d1 = v_perm_b32(hi, lo, 0x05010400), v_perm_b32(hi, lo, 0x07030602)
    assert [(d0 >> (8 * i)) & 0xFF for i in range(4)] == [0, 1, 2, 3]
    assert [(d1 >> (8 * i)) & 0xFF for i in range(4)] == [4, 5, 6, 7]


def lds_swz(row):
    return row & 7


def lds_off(row, chunk):
    return row * 128 + ((chunk ^ lds_swz(row)) << 4)


def test_lds_swizzle_is_a_bijection_and_spreads_banks():
    rows = 256
    offs = {lds_off(r, c) for r in range(rows) for c in range(8)}
    assert len(offs) == rows * 8 and max(offs) == rows * 128 - 16
    # MFMA operand read: a 16-byte read is served 8 lanes at a time, i.e. 8 consecutive rows of one
    # logical chunk; those must land in 8 distinct 16-byte slots of the 128-byte row pitch
    for r0 in range(0, rows, 8):
        for c in range(8):
            assert len({(lds_off(r0 + r, c) % 128) // 16 for r in range(8)}) == 8
    # tile fill: 8 consecutive lanes write the 8 chunks of one row -> 8 distinct slots as well
    for r in range(rows):
        assert len({(lds_off(r, c) % 128) // 16 for c in range(8)}) == 8


def test_five_slot_schedule_keeps_every_tile_until_it_is_read():
    """Restatement of the issue / wait order of gemm_slots_kernel (csrc/gemm_slots.h) for one wavefront: tile t lives
    in slot t % 5 (A of stage s is t = 2s, W is t = 2s + 1); loads retire in issue order, `wait(keep)` guarantees all
    tiles but the youngest when keep is set.  No slot may be reloaded before its tile was multiplied, and every tile
    must be covered by a wait before its stage."""
    def run(KT):
        issued, owner, read = [], {}, set()
        landed = 0

        def issue(name, t):
            prev = owner.get(t % 5)
            assert prev is None or prev in read, (KT, name, "overwrites", prev)
            owner[t % 5] = name
            issued.append(name)

        issue("A0", 0)
        issue("W0", 1)
        if KT > 1:
            issue("A1", 2)
        landed = len(issued) - (1 if KT > 1 else 0)
        for k in range(KT):
            if k + 1 < KT:
                issue(f"W{k + 1}", 2 * k + 3)
            if k + 2 < KT:
                issue(f"A{k + 2}", 2 * k + 4)
            for name, t in ((f"A{k}", 2 * k), (f"W{k}", 2 * k + 1)):
                assert issued.index(name) < landed, (KT, name, "not waited for")
                assert owner[t % 5] == name, (KT, name, "slot taken by", owner[t % 5])
            read.update((f"A{k}", f"W{k}"))
            if k + 1 < KT:
                keep = k + 2 < KT
                assert not keep or issued[-1] == f"A{k + 2}"
                landed = len(issued) - (1 if keep else 0)

    for KT in range(1, 48):
        run(KT)
