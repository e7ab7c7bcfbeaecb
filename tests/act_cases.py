"""Activation rows that pin aion's int8 activation preparation (cpu/kernels/matmul_q_i8.zig:187-203) to the bit,
and block-form identity weights that turn a matmul step into a read-out of the prepared activation.

With a weight whose row n holds code 1 at position n % K (block scale 1.0) and zero codes elsewhere, every other block dot is
an exact integer 0, so C[n] = f32(code[n % K]) * a_scale[block]: one f32 product of the two things the preparation produces.
The q4 form (nibble 9 at the position, 8 = zero elsewhere) also needs the block's code sum to be right, because the
kernels take the -8 offset of the nibbles back as -8 * sum(codes).
"""
import numpy as np

F32 = np.float32


def _bits(u):
    return np.array([u], np.uint32).view(np.float32)[0]


# amax = 127 -> inv = 1 exactly: x.5 are exact ties. Round half away from zero gives 1, 2, 3, -1, -2, -3, 64, -64, 127, -127;
# round half to even would give 0, 2, 2, 0, -2, -2, 64, -64, 126, -126.
TIE_BLOCK = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, 126.49, 0.49999997, -0.49999997, 0.0, 3.5,
             4.5, -4.5, 0.25, -0.75, 100.5, -99.5, 7.0, -8.0, 1e-20, -1e-20, 5.5, 6.5, -7.5, 8.5, 0.0, -0.0]
TIE_CODES = [127, 1, 2, 3, -1, -2, -3, 64, -64, 127, -127, 126, 0, 0, 0, 4,
             5, -5, 0, -1, 101, -100, 7, -8, 0, 0, 6, 7, -8, 9, 0, 0]
# amax = 254 held by a negative element -> inv = 0.5 exactly: odd integers are ties
HALF_BLOCK = [-254.0] + [float(2 * k + 1) * (1 if k % 2 else -1) for k in range(31)]
# 127 / amax and 1 / (amax / 127) differ for this amax, and each of the next four values (and their negatives) gets a
# different code from the two (1, 2, 3, 4 from 127 / amax; 2, 3, 4, 5 from the other): found by a search over f32 values, kept as bit patterns
INV_BLOCK = [_bits(0x40747F5B)] + [s * _bits(b) for b in (0x3D38D126, 0x3D9A03A0, 0x3DD79EAC, 0x3E0A9CDC) for s in (1, -1)]
INV_CODES = [127, 1, -1, 2, -2, 3, -3, 4, -4]


def block_kinds(rng):
    """One block of each kind, in a fixed order."""
    inv = np.zeros(32, F32)
    inv[:len(INV_BLOCK)] = INV_BLOCK
    inv[len(INV_BLOCK):] = rng.uniform(-3.5, 3.5, 32 - len(INV_BLOCK)).astype(F32)
    denormal = (np.array([1e-40], F32)[0] * (1 + np.arange(32) % 5) * np.where(np.arange(32) % 2, -1, 1)).astype(F32)
    tiny = (rng.standard_normal(32) * 1e-30).astype(F32)
    single = np.zeros(32, F32)
    single[17] = -3.25
    return [np.array(TIE_BLOCK, F32), np.zeros(32, F32), np.array(HALF_BLOCK, F32), inv, denormal, tiny, single,
            rng.standard_normal(32).astype(F32), (rng.standard_normal(32) * 1e4).astype(F32)]


def rows(m, k, seed, denormal=True):
    """[m, k] f32: the special blocks cycled along K (shifted by one kind per row), the rest N(0,1).
    denormal=False leaves the denormal-amax block out (for callers that scale the row by a power of two first)."""
    rng = np.random.default_rng(seed)
    out = np.zeros((m, k), F32)
    for r in range(m):
        kinds = block_kinds(rng)
        if not denormal:
            del kinds[4]
        for kb in range(k // 32):
            i = (kb + r) % (len(kinds) + 3)
            out[r, kb * 32:(kb + 1) * 32] = kinds[i] if i < len(kinds) else rng.standard_normal(32).astype(F32)
    return out


def expected_readout(orc, a, n):
    """What the identity weight reads out: f32(code) * scale, for columns n % K."""
    aq, sc, _sm = orc.prepare_a(a)
    full = aq.astype(F32) * np.repeat(sc, 32, axis=1)
    k = a.shape[1]
    return full[:, np.arange(n) % k]


def identity_q8_rows(n, k):
    """q8_0 [N,K] quant_axis 1 (block (n, kb) at (n*K/32+kb)*34): code 1 at position n % K, scale 1.0 everywhere."""
    kb = k // 32
    blocks = np.zeros((n, kb, 34), np.uint8)
    blocks[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    pos = np.arange(n) % k
    blocks[np.arange(n), pos // 32, 2 + pos % 32] = 1
    return blocks.reshape(-1)


def identity_q8_kmajor(n, k):
    """q8_0 [K,N] quant_axis 0 (block (kb, n) at (kb*N+n)*34)."""
    kb = k // 32
    blocks = np.zeros((kb, n, 34), np.uint8)
    blocks[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    pos = np.arange(n) % k
    blocks[pos // 32, np.arange(n), 2 + pos % 32] = 1
    return blocks.reshape(-1)


def identity_q4_kmajor(n, k):
    """q4_0 [K,N] quant_axis 0 (block (kb, n) at (kb*N+n)*18): nibble 9 (= +1) at position n % K, nibble 8 (= 0) elsewhere;
    element t sits in byte t >> 1, low nibble for even t (cpu/test_cpu_kernels.zig:490-523)."""
    kb = k // 32
    blocks = np.full((kb, n, 18), 0x88, np.uint8)
    blocks[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    pos = np.arange(n) % k
    t = pos % 32
    byte = np.where(t % 2 == 0, 0x89, 0x98).astype(np.uint8)
    blocks[pos // 32, np.arange(n), 2 + t // 2] = byte
    return blocks.reshape(-1)
