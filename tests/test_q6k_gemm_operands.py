"""CPU checks of the arithmetic that the Q6_K GEMM kernels (csrc/gemm.hip: gemm_q6k_frag_kernel, gemm_q6k_pc_kernel,
gemm_q6k_tall_kernel) rest on: the split of the int8 scale into two parts whose products with a quant are exact fp16 numbers, the way a quant
is assembled in place as the fp16 number 1024 + q and turned into such a product by one fused multiply-add, and the
map from (chunk, k-step, lane half, slot) of a matrix-core weight fragment to bytes and bits of a 210-byte block.
The last is restated here in numpy and compared with the oracle's dequantization of the same block."""
import numpy as np

from oracle import oracle_np
from skainet_amd import synth

Q6_K = synth.Q6_K


def _exact_f16(v):
    return np.array_equal(np.asarray(v, np.float64), np.asarray(v, np.float64).astype(np.float16).astype(np.float64))


def test_scale_split_gives_exact_fp16_operands_for_every_quant_and_scale():
    q = np.arange(64).reshape(-1, 1) - 32            # q - 32
    sc = np.arange(-128, 128).reshape(1, -1)
    s0, s1 = sc & 15, sc >> 4                        # (arithmetic shift: -8 .. 7)
    assert np.array_equal(16 * s1 + s0, sc)
    assert s0.min() == 0 and s0.max() == 15 and s1.min() == -8 and s1.max() == 7
    part1, part0 = q * s1, q * s0 / 16.0
    assert _exact_f16(part1) and _exact_f16(part0)
    # the two parts through the matrix core into one accumulator: sum = sc (q - 32) / 16, the unit is 16 d
    assert np.array_equal((part1 + part0) * 16.0, (q * sc).astype(np.float64))
    # the product itself does not fit an fp16 operand: that is why there are two parts
    assert not _exact_f16(q * sc)


def test_in_place_assembly_and_the_fused_multiply_add():
    ql = np.arange(16, dtype=np.uint32).reshape(-1, 1)   # low four bits
    qh = np.arange(4, dtype=np.uint32).reshape(1, -1)    # high two bits
    bits = (0x6400 | ql | (qh << 4)).astype(np.uint16)
    val = bits.view(np.float16).astype(np.float64)
    assert np.array_equal(val, 1024.0 + (ql + 16 * qh))  # 0x6400 is 1024 and its last mantissa bit is 1
    for s in list(range(-8, 8)) + [x / 16.0 for x in range(16)]:
        c = -1056.0 * s
        assert _exact_f16(s) and _exact_f16(c)           # 1056 s = 33 s 2^5
        # a fused multiply-add rounds once, after the exact product and sum: (1024 + q) s - 1056 s = (q - 32) s
        got = (val * s + c).astype(np.float16).astype(np.float64)
        assert np.array_equal(got, (ql + 16 * qh - 32.0) * s)


def _fragment_elements(block, c, s, h):
    """The eight weights that lane half h hands to the matrix core for k-step s of chunk c of one superblock, as the
    kernels read them: dword s of three sixteen-byte pieces, shifted right by four for odd chunks."""
    half, par = c >> 1, c & 1
    ql = block[0:128]
    qh = block[128:192]
    scales = block[192:208].view(np.int8)
    d = float(block[208:210].view(np.float16)[0])

    def dword(buf, off):
        return int(np.frombuffer(buf[off:off + 4].tobytes(), dtype="<u4")[0])

    x = dword(ql, 64 * half + 16 * h + 4 * s) >> (4 * par)
    y = dword(ql, 64 * half + 32 + 16 * h + 4 * s) >> (4 * par)
    z = dword(qh, 32 * half + 16 * h + 4 * s) >> (4 * par)
    x8, y8, z8 = x >> 8, y >> 8, z >> 8
    pairs = [((z & 0x00030003) << 4) | (x & 0x000F000F),
             ((z & 0x000C000C) << 2) | (y & 0x000F000F),
             ((z8 & 0x00030003) << 4) | (x8 & 0x000F000F),
             ((z8 & 0x000C000C) << 2) | (y8 & 0x000F000F)]
    sc_lo, sc_hi = int(scales[4 * c + h]), int(scales[4 * c + 2 + h])   # bytes h and 2 + h of dword c of the scales
    out = []
    for e, p in enumerate(pairs):
        sc = sc_lo if e % 2 == 0 else sc_hi
        for q in (p & 0xFFFF, p >> 16):
            out.append(d * sc * (q - 32))
    return out


def test_fragment_map_reads_the_elements_the_activation_fragments_hold():
    raw = synth.weight(Q6_K, 3, 256, seed=5).reshape(3, 210).copy()
    rng = np.random.default_rng(6)
    raw[:, 192:208] = rng.integers(-128, 128, size=(3, 16), dtype=np.int8).view(np.uint8)
    want = oracle_np.dequant(Q6_K, raw.reshape(-1)).reshape(3, 256).astype(np.float64)
    for b in range(3):
        for c in range(4):
            for s in range(4):
                for h in range(2):
                    dw = 4 * h + s
                    # the element order of an activation fragment inside its chunk of 64
                    idx = [4 * dw + 0, 4 * dw + 2, 32 + 4 * dw + 0, 32 + 4 * dw + 2,
                           4 * dw + 1, 4 * dw + 3, 32 + 4 * dw + 1, 32 + 4 * dw + 3]
                    got = _fragment_elements(raw[b], c, s, h)
                    exp = [want[b, 64 * c + i] for i in idx]
                    assert np.allclose(got, exp, rtol=1e-6, atol=0.0), (b, c, s, h)
