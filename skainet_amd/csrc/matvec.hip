// Batch-1 quantized matvec  y[n] = sum_k deq(W)[n,k] * x[k]  for GGUF Q4_K, Q8_0 and Q6_K weights, and -- on the
// Q4_K kernel's lane map -- Q5_K, Q4_0, Q4_1, Q5_0, Q5_1 and IQ4_NL; the fused forms the decoder uses (norm folded into the
// staging of x, several matrices per launch, residual / SwiGLU / rotary + cache-store epilogues) for all of these.
//
// The op is bound by the HBM read of the weight blocks (0.5625 / 1.0625 / 0.8203 bytes per weight for the first
// three); x is read once per workgroup and y written once.  One wavefront owns one output row, so the only
// cross-lane traffic is a single DPP reduction per row and rows never need atomics.
#include "kv.h"
#include <type_traits>

namespace {

// ------------------------------------------------------------------------------------------ Q4_K
//
// A row of k weights is k/256 superblocks of 144 bytes = 9 aligned 16-byte chunks each: one header chunk
// (f16 d, f16 dmin, 12 bytes of 6-bit scales/mins) and eight chunks of nibbles.  Per step a wavefront takes
// sixteen superblocks of R consecutive rows: lane (b, p) = (lane / 4, lane % 4) owns the 64 weights of
// sub-block pair p of superblock b -- nibble chunks 2p and 2p+1, two 128-bit loads -- plus the header chunk
// that its four lanes share.  Every load of the wavefront's rows is issued before anything is consumed.
//
// Nibble bytes 32p..32p+31 of qs: low nibbles are elements 64p + 0..31 (sub-block 2p), high nibbles elements
// 64p + 32..63 (sub-block 2p+1).  The activation is staged in LDS in lane order -- slot [(step*16 + i)*64 + lane]
// is the i-th float4 of the lane's 64 activations -- so the 128-bit LDS reads are conflict-free, and one read
// of x serves the R rows.  Two tricks keep the VALU work per weight low:
//   * a nibble masked in place (q & 0x000F000F, q & 0x00F000F0) is read as a pair of fp16 subnormals
//     n * 2^-24 (or 16n * 2^-24), which v_fma_mix_f32 multiplies with the fp32 activation directly: no
//     integer-to-float conversion, one mask per two weights, one fused multiply-add per weight;
//   * the powers of two are folded in where they cost least: a high nibble is read sixteen-fold, so the scale of
//     its sub-block is divided by 16 (once per lane and step; x itself is staged as it is), the per-sub-block
//     sums of x (for the "- dmin * m" term) are multiplied by 2^-24 in the staging, and the row total is
//     multiplied by 2^24 once.
//
//   y = 2^24 * sum_blocks [ d * (sc_lo * A_lo + sc_hi * A_hi) - dmin * (m_lo * S_lo + m_hi * S_hi) ]

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// 16 loaded bytes as a native vector: the value stays one four-register tuple from the load to its use.  With
// HIP's uint4 (a struct) the four words are split at the load and the register allocator parks and re-copies
// them, which puts a wait for the load in front of each copy.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// LDS pitch (in float4) of one row of 64 lane slots: 65 puts the sixteen float4 of one column, which the staging
// stores write from sixteen consecutive lanes, into different banks; the per-lane reads stay contiguous.
constexpr int kXPitch = 65;

// 6-bit scales / mins of sub-blocks 2p and 2p+1 out of the header chunk h = (d|dmin, scales[0..3], [4..7], [8..11]).
// Branch-free and two values at a time: both packings are formed as byte pairs and the lane's pair index
// selects one, so the header registers are only ever read by straight-line code.
__device__ __forceinline__ void q4k_pair_scales(const u32x4& h, int pair, float& sc0, float& sc1, float& m0,
                                                float& m1) {
    const int sh = 16 * (pair & 1);
    const uint32_t a = h.y >> sh, b = h.z >> sh, c = h.w >> sh;
    const uint32_t s_lo = a & 0x3F3Fu, n_lo = b & 0x3F3Fu;                        // sub-blocks 0..3: plain 6-bit fields
    const uint32_t s_hi = (c & 0x0F0Fu) | ((a >> 2) & 0x3030u);                    // sub-blocks 4..7: 4 low bits in
    const uint32_t n_hi = ((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);             // scales[8..11], 2 high bits parked
    const uint32_t sp = pair < 2 ? s_lo : s_hi;                                    // in the tops of scales[0..7]
    const uint32_t np = pair < 2 ? n_lo : n_hi;
    sc0 = (float)(sp & 0xFF);
    sc1 = (float)((sp >> 8) & 0xFF);
    m0 = (float)(np & 0xFF);
    m1 = (float)((np >> 8) & 0xFF);
}

// One dword of nibbles: low nibbles of bytes 0..3 against xl.{x,y,z,w}, high nibbles against xh (pre-divided by 16).
__device__ __forceinline__ void q4k_dot_dword(uint32_t q, const float4& xl, const float4& xh, float& alo, float& ahi) {
    const uint32_t q8 = q >> 8;
    const half2_t l02 = __builtin_bit_cast(half2_t, q & 0x000F000Fu);
    const half2_t h02 = __builtin_bit_cast(half2_t, q & 0x00F000F0u);
    const half2_t l13 = __builtin_bit_cast(half2_t, q8 & 0x000F000Fu);
    const half2_t h13 = __builtin_bit_cast(half2_t, q8 & 0x00F000F0u);
    alo = fmaf((float)l02.x, xl.x, alo);
    ahi = fmaf((float)h02.x, xh.x, ahi);
    alo = fmaf((float)l13.x, xl.y, alo);
    ahi = fmaf((float)h13.x, xh.y, ahi);
    alo = fmaf((float)l02.y, xl.z, alo);
    ahi = fmaf((float)h02.y, xh.z, ahi);
    alo = fmaf((float)l13.y, xl.w, alo);
    ahi = fmaf((float)h13.y, xh.w, ahi);
}

// Q5_K: the same dword of nibbles with the dword of qh that holds the fifth bits of its four elements, already
// shifted so that bit 0 of each byte belongs to the low-nibble sub-block and bit 1 to the high-nibble one.  The
// fifth bit joins its nibble before the multiply (bit 4 of the low value, bit 8 of the sixteen-fold high value),
// so the fp16 subnormal read by v_fma_mix_f32 is the whole five-bit quant.
__device__ __forceinline__ void q5k_dot_dword(uint32_t q, uint32_t hq, const float4& xl, const float4& xh, float& alo,
                                              float& ahi) {
    const uint32_t q8 = q >> 8, hq8 = hq >> 8;
    const half2_t l02 = __builtin_bit_cast(half2_t, (q & 0x000F000Fu) | ((hq & 0x00010001u) << 4));
    const half2_t h02 = __builtin_bit_cast(half2_t, (q & 0x00F000F0u) | ((hq & 0x00020002u) << 7));
    const half2_t l13 = __builtin_bit_cast(half2_t, (q8 & 0x000F000Fu) | ((hq8 & 0x00010001u) << 4));
    const half2_t h13 = __builtin_bit_cast(half2_t, (q8 & 0x00F000F0u) | ((hq8 & 0x00020002u) << 7));
    alo = fmaf((float)l02.x, xl.x, alo);
    ahi = fmaf((float)h02.x, xh.x, ahi);
    alo = fmaf((float)l13.x, xl.y, alo);
    ahi = fmaf((float)h13.x, xh.y, ahi);
    alo = fmaf((float)l02.y, xl.z, alo);
    ahi = fmaf((float)h02.y, xh.z, ahi);
    alo = fmaf((float)l13.y, xl.w, alo);
    ahi = fmaf((float)h13.y, xh.w, ahi);
}

// Staging of x, split in two so that the weight loads can be issued in between: coalesced global loads
// (thread t takes float4 t, t + blockDim, ...: a wavefront reads 1 KiB contiguous per instruction) into
// registers, and later the LDS stores, which do the transposition into lane order.  float4 f of x belongs to
// column f / 16 (64 activations of one (superblock, pair)), position f % 16 in it; the eight threads that
// hold one half column are eight consecutive lanes, so its sum is a DPP reduction.
template <int J>
struct Q4kStage {
    float4 v[J];
};

template <int J>
__device__ __forceinline__ void q4k_stage_load(const float* __restrict__ x, int n4, int tid, int nthreads,
                                               Q4kStage<J>& st) {
    const float4* x4 = reinterpret_cast<const float4*>(x);
#pragma unroll
    for (int j = 0; j < J; j++) st.v[j] = x4[min(tid + j * nthreads, n4 - 1)];
}

// Q4K: the half-column sums carry the 2^-24 of the Q4_K kernel's nibble units.  Otherwise (Q8_0): they are
// multiplied by 128, the offset that turns the signed quants into unsigned bytes.  x is stored as it is.
// HI: kept for the callers' sake (the bit of a float4's position that tells a high-nibble one); unused since the
// sixteen-fold reading of high nibbles is undone in the scales instead of in the staged x.
template <bool Q4K = true, int HI = 8>
__device__ __forceinline__ void q4k_stage_store_one(const float4& v, int f, float4* xs, float* ss) {
    const int cc = f >> 4, i16 = f & 15;
    const int step = cc >> 6, ln = cc & 63;
    xs[(step * 16 + i16) * kXPitch + ln] = v;
    float sum = (v.x + v.y) + (v.z + v.w);
    sum += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sum), 0xB1, 0xF, 0xF, true));   // lane ^ 1
    sum += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sum), 0x4E, 0xF, 0xF, true));   // lane ^ 2
    sum += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sum), 0x141, 0xF, 0xF, true));  // 7 - lane
    if ((f & 7) == 0) ss[f >> 3] = sum * (Q4K ? 5.9604644775390625e-08f : 128.0f);  // 2^-24, see the scaling note above
}

template <int J, bool Q4K = true, int HI = 8>
__device__ __forceinline__ void q4k_stage_store(const Q4kStage<J>& st, int n4, int tid, int nthreads, float4* xs,
                                                float* ss) {
#pragma unroll
    for (int j = 0; j < J; j++) {
        // a float4 index past the end repeats the last one: same data to the same slot (no branch; whole
        // groups of eight lanes are clamped together because n4 is a multiple of 64)
        const int f = min(tid + j * nthreads, n4 - 1);
        q4k_stage_store_one<Q4K, HI>(st.v[j], f, xs, ss);
    }
}

struct Q4kLoads {
    u32x4 h, qa, qb;
    bool ok;  // false: the slot lies past the row end / past the last row and must contribute nothing
};

// Q5_K (176 bytes: header chunk, two chunks of qh, eight of qs): the 32 bytes of fifth bits as well -- bit j of
// qh[l] belongs to element l of sub-block j, so every lane of a superblock needs all of them
struct Q5kLoads : Q4kLoads {
    u32x4 ha, hb;
};

// The formats with blocks of 32 on the same lane map: eight blocks stand where a superblock stands, lane (sub, p)
// takes blocks 2p and 2p + 1 of its eight -- 36 to 48 contiguous bytes at 4-byte alignment, nine to twelve dwords.
//   Q4_0 (18 bytes: f16 d, 16 bytes of nibbles; low nibbles are elements 0..15, high nibbles 16..31; d (q - 8)):
//     dword 0 = d | q0 q1, dwords 1..3, dword 4 = q14 q15 | d', dwords 5..8 the second block's nibbles; the first
//     block's are realigned with v_alignbyte.
//   Q4_1 (20 bytes: d, f16 m, nibbles; d q + m): every field is an aligned dword.
//   Q5_0 (22 bytes: d, four bytes of fifth bits -- bit e of the dword belongs to element e --, nibbles; d (q - 16)):
//     first block realigned (fifth bits and nibbles), second block aligned from dword 6.
//   Q5_1 (24 bytes: d, m, fifth bits, nibbles; d q + m): aligned.
// The four fifth bits that go with a dword of nibbles are spread to bit 0 of its four bytes by one multiply
// ((bits * 0x00204081) & 0x01010101: bit k lands on 8k, no two partial products meet), those of the high nibbles
// to bit 1, which is the form q5k_dot_dword takes.
constexpr int kFmtQ4K = 0, kFmtQ5K = 1, kFmtQ40 = 2, kFmtQ41 = 3, kFmtQ50 = 4, kFmtQ51 = 5, kFmtIQ4NL = 8, kFmtIQ4XS = 9;
constexpr int kFmtQ6K = 6, kFmtQ80 = 7;  // (fused kernels only: the lane maps, staging and steps of matvec_q6k_kernel / matvec_q80_pairs_kernel)
constexpr int kFmtQ2K = 10, kFmtQ3K = 11, kFmtQ8K = 12, kFmtTQ2 = 13, kFmtTQ1 = 14;  // (fused kernels only: those of matvec_runs_kernel / matvec_q8k_kernel / matvec_tq1_kernel)
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x3_a4 __attribute__((ext_vector_type(3), aligned(4)));
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

struct Q4xLoads {
    u32x4 a, b, c;  // dwords 0..11 (c: as many as the format has)
    bool ok;
};

//   IQ4_NL (18 bytes, the layout of Q4_0; d table[q] with sixteen signed values): four nibbles at a time are looked
//     up with two v_perm_b32 (entries 0..7 and 8..15) and a bit select on bit 3; the table holds value + 128, so
//     the bytes are unsigned for v_cvt_f32_ubyteN and the 128 comes back out as 128 sum(x of the block), which the
//     staging forms (x itself is staged unscaled for this format).
__device__ __forceinline__ uint32_t iq4nl_lookup4(uint32_t idx) {  // idx: four table indices, one per byte
    // -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113, each plus 128
    constexpr uint32_t T0 = 0x3F2D1801u, T1 = 0x766A5D4Fu, T2 = 0xA6998D81u, T3 = 0xF1D9C5B5u;
    const uint32_t sel = idx & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel), hi = __builtin_amdgcn_perm(T3, T2, sel);
    const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}

__device__ __forceinline__ float iq4nl_dot4(uint32_t t, const float4& x, float s) {
    s = fmaf((float)(t & 0xFFu), x.x, s);
    s = fmaf((float)((t >> 8) & 0xFFu), x.y, s);
    s = fmaf((float)((t >> 16) & 0xFFu), x.z, s);
    s = fmaf((float)(t >> 24), x.w, s);
    return s;
}

//   IQ4_XS (136 bytes per 256: f16 d, u16 scales_h, scales_l[4], qs[128]; 8-byte aligned): a superblock of eight
//     sub-blocks of 32 with the element order and the table of IQ4_NL, so lane (sub, p) takes sub-blocks 2p and 2p + 1
//     as it takes blocks 2p and 2p + 1 there: their 32 bytes of qs (two 16-byte vectors) and the eight header bytes.
//     Scale of sub-block ib: nibble ib % 2 of scales_l[ib / 2] with bits 2 ib, 2 ib + 1 of scales_h on top, minus 32.
__device__ __forceinline__ void iq4xs_load(const uint8_t* block, int p, Q4xLoads& L) {
    L.a = *reinterpret_cast<const u32x4_a4*>(block + 8 + 32 * p);
    L.b = *reinterpret_cast<const u32x4_a4*>(block + 24 + 32 * p);
    const u32x2_a4 t = *reinterpret_cast<const u32x2_a4*>(block);
    L.c = u32x4{t.x, t.y, 0u, 0u};
}

// the lane's two blocks: two 16-byte vectors and the format's tail of one to four dwords
template <int F>
__device__ __forceinline__ void q4x_load(const uint8_t* bp, Q4xLoads& L) {
    L.a = *reinterpret_cast<const u32x4_a4*>(bp);
    L.b = *reinterpret_cast<const u32x4_a4*>(bp + 16);
    L.c = u32x4{0u, 0u, 0u, 0u};
    if (F == kFmtQ40 || F == kFmtIQ4NL) {
        L.c.x = *reinterpret_cast<const uint32_t*>(bp + 32);
    } else if (F == kFmtQ41) {
        const u32x2_a4 t = *reinterpret_cast<const u32x2_a4*>(bp + 32);
        L.c.x = t.x, L.c.y = t.y;
    } else if (F == kFmtQ50) {
        const u32x3_a4 t = *reinterpret_cast<const u32x3_a4*>(bp + 32);
        L.c.x = t.x, L.c.y = t.y, L.c.z = t.z;
    } else {
        L.c = *reinterpret_cast<const u32x4_a4*>(bp + 32);
    }
}

// the fields of the lane's first (half 0) or second block: nibble dwords, fifth bits, scale and offset
template <int F>
__device__ __forceinline__ void q4x_fields(const Q4xLoads& L, int half, int p, uint32_t (&q)[4], uint32_t& qh, float& d, float& m) {
    const u32x4 &a = L.a, &b = L.b, &c = L.c;
    auto lo16 = [](uint32_t w) { return (float)__builtin_bit_cast(half2_t, w).x; };
    auto hi16 = [](uint32_t w) { return (float)__builtin_bit_cast(half2_t, w).y; };
    auto al = [](uint32_t hi, uint32_t lo) { return __builtin_amdgcn_alignbyte(hi, lo, 2); };
    qh = 0u, m = 0.f;
    if (F == kFmtIQ4XS) {
        const u32x4& v = half == 0 ? a : b;
        q[0] = v.x, q[1] = v.y, q[2] = v.z, q[3] = v.w;
        const int ib = 2 * p + half;
        const int ls = (int)(((c.y >> (8 * p + 4 * half)) & 0xFu) | ((((c.x >> 16) >> (2 * ib)) & 3u) << 4)) - 32;
        d = lo16(c.x) * (float)ls;
    } else if (F == kFmtQ40 || F == kFmtIQ4NL) {
        if (half == 0) q[0] = al(a.y, a.x), q[1] = al(a.z, a.y), q[2] = al(a.w, a.z), q[3] = al(b.x, a.w), d = lo16(a.x);
        else q[0] = b.y, q[1] = b.z, q[2] = b.w, q[3] = c.x, d = hi16(b.x);
    } else if (F == kFmtQ41) {
        if (half == 0) q[0] = a.y, q[1] = a.z, q[2] = a.w, q[3] = b.x, d = lo16(a.x), m = hi16(a.x);
        else q[0] = b.z, q[1] = b.w, q[2] = c.x, q[3] = c.y, d = lo16(b.y), m = hi16(b.y);
    } else if (F == kFmtQ50) {
        if (half == 0) qh = al(a.y, a.x), q[0] = al(a.z, a.y), q[1] = al(a.w, a.z), q[2] = al(b.x, a.w), q[3] = al(b.y, b.x), d = lo16(a.x);
        else qh = b.z, q[0] = b.w, q[1] = c.x, q[2] = c.y, q[3] = c.z, d = hi16(b.y);
    } else {
        if (half == 0) qh = a.y, q[0] = a.z, q[1] = a.w, q[2] = b.x, q[3] = b.y, d = lo16(a.x), m = hi16(a.x);
        else qh = b.w, q[0] = c.x, q[1] = c.y, q[2] = c.z, q[3] = c.w, d = lo16(b.z), m = hi16(b.z);
    }
}

template <int R, int F>
__device__ __forceinline__ void q4x_step(const Q4xLoads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, float (&acc)[R]) {
    constexpr bool kFive = F == kFmtQ50 || F == kFmtQ51, kTable = F == kFmtIQ4NL || F == kFmtIQ4XS;
    // the quant that stands for zero (IQ4_NL: the staged sums already carry the 128 of the table)
    constexpr float kZero = F == kFmtQ40 ? -8.0f : (F == kFmtQ50 ? -16.0f : (kTable ? -1.0f : 0.0f));
    const float2 sx = reinterpret_cast<const float2*>(ss)[s * 64 + lane];  // the sums of x over the two blocks (x 2^-24)
    float v[R];
#pragma unroll
    for (int r = 0; r < R; r++) v[r] = 0.f;
#pragma unroll
    for (int half = 0; half < 2; half++) {  // the lane's first and second block
        float4 xl[4], xh[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xl[j] = xs[(s * 16 + 8 * half + j) * kXPitch + lane];
            xh[j] = xs[(s * 16 + 8 * half + 4 + j) * kXPitch + lane];
        }
        const float sxb = half == 0 ? sx.x : sx.y;
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t q[4], qh;
            float d, m;
            q4x_fields<F>(L[r], half, lane & 3, q, qh, d, m);
            float alo = 0.f, ahi = 0.f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (kTable) {
                    alo = iq4nl_dot4(iq4nl_lookup4(q[i] & 0x0F0F0F0Fu), xl[i], alo);
                    ahi = iq4nl_dot4(iq4nl_lookup4((q[i] >> 4) & 0x0F0F0F0Fu), xh[i], ahi);
                } else if (kFive) {
                    const uint32_t lo = (((qh >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u;
                    const uint32_t hi = (((qh >> (16 + 4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u;
                    q5k_dot_dword(q[i], lo | (hi << 1), xl[i], xh[i], alo, ahi);
                } else {
                    q4k_dot_dword(q[i], xl[i], xh[i], alo, ahi);
                }
            }
            const float both = kTable ? alo + ahi : fmaf(ahi, 0.0625f, alo);  // (high nibbles read sixteen-fold)
            v[r] = fmaf(d, fmaf(kZero, sxb, both), fmaf(m, sxb, v[r]));
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] += L[r].ok ? v[r] : 0.f;
}

template <typename LT>
constexpr bool kIsQ5 = false;
template <>
constexpr bool kIsQ5<Q5kLoads> = true;

// One step for R rows: the lane's 64 activations are read from LDS in two halves of 32 (8 float4 live at a
// time) and each half meets the matching nibble chunk of every row.
template <int R, typename LT>
__device__ __forceinline__ void q4k_step(const LT (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, int pair, float (&acc)[R]) {
    float alo[R], ahi[R];
#pragma unroll
    for (int r = 0; r < R; r++) alo[r] = ahi[r] = 0.f;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        float4 xl[4], xh[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xl[j] = xs[(s * 16 + 4 * half + j) * kXPitch + lane];
            xh[j] = xs[(s * 16 + 8 + 4 * half + j) * kXPitch + lane];
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const u32x4 qq = half == 0 ? L[r].qa : L[r].qb;
            if constexpr (kIsQ5<LT>) {
                const u32x4 hh = (half == 0 ? L[r].ha : L[r].hb) >> (uint32_t)(2 * pair);
                q5k_dot_dword(qq.x, hh.x, xl[0], xh[0], alo[r], ahi[r]);
                q5k_dot_dword(qq.y, hh.y, xl[1], xh[1], alo[r], ahi[r]);
                q5k_dot_dword(qq.z, hh.z, xl[2], xh[2], alo[r], ahi[r]);
                q5k_dot_dword(qq.w, hh.w, xl[3], xh[3], alo[r], ahi[r]);
            } else {
                q4k_dot_dword(qq.x, xl[0], xh[0], alo[r], ahi[r]);
                q4k_dot_dword(qq.y, xl[1], xh[1], alo[r], ahi[r]);
                q4k_dot_dword(qq.z, xl[2], xh[2], alo[r], ahi[r]);
                q4k_dot_dword(qq.w, xl[3], xh[3], alo[r], ahi[r]);
            }
        }
    }
    const float2 sx = reinterpret_cast<const float2*>(ss)[s * 64 + lane];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float sc0, sc1, m0, m1;
        q4k_pair_scales(L[r].h, pair, sc0, sc1, m0, m1);
        const uint32_t dword0 = L[r].h.x;  // by value: a bit cast of a vector element reads the whole vector's start
        const half2_t dd = __builtin_bit_cast(half2_t, dword0);
        const float t1 = fmaf(sc1 * 0.0625f, ahi[r], sc0 * alo[r]);  // (the high nibbles were read sixteen-fold)
        const float t2 = fmaf(m1, sx.y, m0 * sx.x);
        const float v = fmaf((float)dd.x, t1, -((float)dd.y * t2));
        acc[r] += L[r].ok ? v : 0.f;
    }
}

// R = consecutive rows per wavefront (x is read from LDS once for the R rows).
// STEPS > 0: the row takes exactly STEPS steps, fully unrolled.  STEPS == 0: rolled loop for any k.
//
// Order of events in a wavefront: issue the x loads, issue the weight loads of step 0, wait for x only (its
// loads are the oldest in flight), store it to LDS, barrier; then per step: issue the weight loads of the
// next step, consume the current one.  A compute unit's memory pipeline accepts only so many requests before
// a wavefront stalls at issue, so the loads are kept one step ahead instead of all up front -- otherwise the
// x stores (and with them every wavefront at the barrier) would sit behind the issue of a whole row.
// F: Q4_K; Q5_K blocks (eleven chunks, the quants from the fourth on) with the same lane map, staging and scales;
// Q4_0 / Q4_1, eight blocks for a superblock (nb counts groups of eight).
// TS: a measuring build (skn_test_matvec_q4k_stamps).  Every wavefront records the wall clock (100 MHz) at its start,
// after its first requests are issued, after its x stores, after the barrier and after each step, plus its hardware
// ids, into the buffer g_matvec_stamps points at: eight 64-bit words per wavefront.  The shipped instantiations have
// TS = false and contain none of it.
__device__ unsigned long long* g_matvec_stamps = nullptr;

template <int STEPS, int R, int F = kFmtQ4K, bool TS = false>
__global__ __launch_bounds__(512) void matvec_q4k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                         float* __restrict__ y, int n_rows, int nb) {
    unsigned long long ts[8] = {};
    if constexpr (TS) ts[0] = wall_clock64();
    constexpr bool Q5 = F == kFmtQ5K, kSmall = F >= kFmtQ40, kXS = F == kFmtIQ4XS;
    using Loads = std::conditional_t<kSmall, Q4xLoads, std::conditional_t<Q5, Q5kLoads, Q4kLoads>>;
    constexpr int kChunks = Q5 ? 11 : 9, kFirst = Q5 ? 3 : 1;  // chunks per block, first chunk of quants
    constexpr int kSmallBytes = (F == kFmtQ40 || F == kFmtIQ4NL) ? 18 : (F == kFmtQ41 ? 20 : (F == kFmtQ50 ? 22 : 24)), kHi = kSmall ? 4 : 8;
    constexpr bool kPlainX = F == kFmtIQ4NL || kXS;  // x staged unscaled, block sums times 128, results in true units
    extern __shared__ float4 lds4[];
    const int steps = STEPS > 0 ? STEPS : (nb + 15) >> 4;
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + steps * 16 * kXPitch);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = blockDim.x >> 6;
    const int row0 = (blockIdx.x * waves + wave) * R;
    const int sub = lane >> 2;  // superblock within the step
    const int p = lane & 3;     // sub-block pair within the superblock
    // bytes of a row (eight small blocks: 8 * kSmallBytes)
    const size_t row_bytes = kXS ? (size_t)nb * 136 : kSmall ? (size_t)nb * (8 * kSmallBytes) : (size_t)nb * (16 * kChunks);
    const int n4 = nb * 64;  // float4 count of x

    // the first J float4 per thread go into registers now; J covers all of x in the unrolled kernels
    // (the launcher runs them with 512 threads: 2 * STEPS * 512 float4 >= k / 4)
    constexpr int J = STEPS > 0 ? 2 * STEPS : 2;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, blockDim.x, st);

    float acc[R];
    const u32x4* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        // slots past the end of a row / past the last row read valid memory (clamped) and are masked at the end
        rp[r] = reinterpret_cast<const u32x4*>(w + (size_t)min(row0 + r, n_rows - 1) * row_bytes) + (kSmall ? 0 : kFirst + 2 * p);
    }
    auto issue = [&](int s, int tie, Loads (&L)[R]) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if constexpr (kXS) {
                iq4xs_load(reinterpret_cast<const uint8_t*>(rp[r]) + (size_t)min(blk, nb - 1) * 136 + tie, p, L[r]);
            } else if constexpr (kSmall) {
                const uint8_t* bp = reinterpret_cast<const uint8_t*>(rp[r]) + (size_t)(min(blk, nb - 1) * 8 + 2 * p) * kSmallBytes + tie;
                q4x_load<F>(bp, L[r]);
            } else {
                const u32x4* bp = rp[r] + min(blk, nb - 1) * kChunks + tie;
                L[r].qa = bp[0];
                L[r].qb = bp[1];
                L[r].h = bp[-kFirst - 2 * p];
                if constexpr (Q5) {
                    L[r].ha = bp[1 - kFirst - 2 * p];
                    L[r].hb = bp[2 - kFirst - 2 * p];
                }
            }
            L[r].ok = row_ok[r] && blk < nb;
        }
    };
    auto step = [&](const Loads (&L)[R], int s, int ln) __attribute__((always_inline)) {
        if constexpr (kSmall) q4x_step<R, F>(L, xs, ss, s, ln, acc);
        else q4k_step<R>(L, xs, ss, s, ln, p, acc);
    };

    if constexpr (STEPS > 0) {
        Loads L[STEPS][R];
        issue(0, 0, L[0]);
        if constexpr (TS) {
            asm volatile("" ::: "memory");
            ts[1] = wall_clock64();
        }
        q4k_stage_store<J, !kPlainX, kHi>(st, n4, tid, blockDim.x, xs, ss);
        if constexpr (TS) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            ts[2] = wall_clock64();
        }
        __syncthreads();
        if constexpr (TS) ts[3] = wall_clock64();
        // `tie` is always 0; an empty asm after each step makes it look rewritten from the finished accumulator,
        // which pins the loads of step s+1 between the arithmetic of steps s-1 and s (one step of lookahead) and
        // the LDS reads of step s below the arithmetic of step s-1 (bounded registers)
        int tie = 0;
        asm volatile("" : "+v"(tie));
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            if (s + 1 < STEPS) issue(s + 1, tie, L[s + 1]);
            asm volatile("" ::: "memory");  // the loads above stay above the LDS reads below
            step(L[s], s, lane + tie);
            asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
            if constexpr (TS && STEPS <= 3) ts[4 + s] = wall_clock64();
        }
        if constexpr (TS) {
            // hardware ids: HW_ID (wave, SIMD, compute unit, shader array, shader engine) and XCC_ID
            ts[7] = ((unsigned long long)__builtin_amdgcn_s_getreg(63508) << 32) | (unsigned)__builtin_amdgcn_s_getreg(63492);
            if (lane == 0 && g_matvec_stamps) {
#pragma unroll
                for (int i = 0; i < 8; i++) g_matvec_stamps[(size_t)(blockIdx.x * waves + wave) * 8 + i] = ts[i];
            }
        }
    } else {
        Loads bufa[R], bufb[R];
        issue(0, 0, bufa);
        q4k_stage_store<J, !kPlainX, kHi>(st, n4, tid, blockDim.x, xs, ss);
        for (int f = tid + J * blockDim.x; f < n4; f += blockDim.x)
            q4k_stage_store_one<!kPlainX, kHi>(reinterpret_cast<const float4*>(x)[f], f, xs, ss);
        __syncthreads();
        for (int s = 0; s < steps; s += 2) {
            if (s + 1 < steps) issue(s + 1, 0, bufb);
            step(bufa, s, lane);
            if (s + 1 < steps) {
                if (s + 2 < steps) issue(s + 2, 0, bufa);
                step(bufb, s + 1, lane);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]) * (kPlainX ? 1.0f : 16777216.0f);
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// The same arithmetic with k split across workgroups: workgroup (g, s) takes rows R * 8 g .. and the s-th step of
// sixteen superblocks, stages only that 4096-slice of x (17 KB of LDS instead of the whole vector, so four workgroups
// and 32 wavefronts fit a compute unit) and leaves one partial per row.  MERGE 1: the partials go to a scratch array
// and the workgroup that takes a row group's last ticket adds them in slice order (deterministic; the counters return
// to zero).  MERGE 2: they are added into y with floating-point atomics (y zeroed by the caller; the order of the
// additions, and with it the last bit, varies).  Measured slower than whole rows per wavefront at every shape tried --
// a launch of 1.5 rounds of workgroups pays the latency to first data twice, and the ticket costs two more round
// trips -- and therefore not the default (option q4k.split; profiles/matvec_q4k_4096x11008.md has the figures).
template <int R, int MERGE>
__global__ __launch_bounds__(512) void matvec_q4k_split_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                               float* __restrict__ y, int n_rows, int nb, int n_slices,
                                                               float* part, int* tickets) {
    __shared__ float4 xs[16 * kXPitch];
    __shared__ float ss[128];
    __shared__ int last_flag;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = blockIdx.x / n_slices, s = blockIdx.x - g * n_slices;
    const int sub = lane >> 2, p = lane & 3;
    const int n4 = nb * 64;
    Q4kStage<2> st;
    {
        const float4* x4 = reinterpret_cast<const float4*>(x);
#pragma unroll
        for (int j = 0; j < 2; j++) st.v[j] = x4[min(s * 1024 + tid + j * 512, n4 - 1)];
    }
    const int row0 = (g * 8 + wave) * R;
    const int blk = s * 16 + sub;
    Q4kLoads L[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const u32x4* bp = reinterpret_cast<const u32x4*>(w + (size_t)min(row0 + r, n_rows - 1) * nb * 144) + min(blk, nb - 1) * 9;
        L[r].qa = bp[1 + 2 * p];
        L[r].qb = bp[2 + 2 * p];
        L[r].h = bp[0];
        L[r].ok = row0 + r < n_rows && blk < nb;
    }
    // local float4 f of the slice goes where float4 f of a whole vector's first step goes (a float4 past the end of x
    // repeats the last one; its superblock is masked)
    q4k_stage_store<2>(st, 1024, tid, 512, xs, ss);
    __syncthreads();
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    q4k_step<R>(L, xs, ss, 0, lane, p, acc);
    float tot[R];
#pragma unroll
    for (int r = 0; r < R; r++) tot[r] = wave_sum(acc[r]) * 16777216.0f;
    if (n_slices == 1) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; r++)
                if (row0 + r < n_rows) y[row0 + r] = tot[r];
        }
        return;
    }
    if (MERGE == 2) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; r++)
                if (row0 + r < n_rows) atomicAdd(&y[row0 + r], tot[r]);
        }
        return;
    }
    // partials and tickets as device-scope atomics, the stores waited for before the ticket is taken (the hand-off of
    // the decode attention's split merge)
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (row0 + r < n_rows) __hip_atomic_store(&part[(size_t)s * n_rows + row0 + r], tot[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) last_flag = __hip_atomic_fetch_add(&tickets[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_slices - 1;
    __syncthreads();
    if (!last_flag) return;
    if (tid < 8 * R) {
        const int row = g * 8 * R + tid;
        if (row < n_rows) {
            float sum = 0.f;
            for (int i = 0; i < n_slices; i++) sum += __hip_atomic_load(&part[(size_t)i * n_rows + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            y[row] = sum;
        }
    }
    if (tid == 0) __hip_atomic_store(&tickets[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------------------ Q8_0
//
// 34-byte blocks (f16 d, 32 x int8), only 2-byte aligned.  Two consecutive blocks are 68 bytes = 17 dwords:
//   dword 0 = d0 | q0 q1, dwords 1..7 = q2..q29, dword 8 = q30 q31 | d1, dwords 9..16 = the 32 quants of the
// second block.  When the row is a whole number of pairs and 4-byte aligned, lane l of a step takes pair
// 64 * step + l (four 16-byte loads and one dword at 4-byte alignment): the second block's quants are aligned
// dwords, the first block's are realigned with v_alignbyte.  Signed bytes become unsigned by flipping the top
// bit (q + 128), which v_cvt_f32_ubyteN converts with the byte select built in: one convert and one fused
// multiply-add per weight; the offset comes back out as 128 * sum(x of the block), formed once per workgroup
// while x is staged.  Staging, lookahead and reduction are those of the Q4_K kernel (a lane's 64 activations
// are the same 64 consecutive elements there and here).
struct Q80Loads {
    u32x4 w[4];    // dwords 0..15
    uint32_t w16;  // dword 16
    bool ok;
};

__device__ __forceinline__ float q80_dot_dword(uint32_t q, const float4& x, float s) {
    const uint32_t u = q ^ 0x80808080u;
    s = fmaf((float)(u & 0xFF), x.x, s);          // (each of these is one v_cvt_f32_ubyteN)
    s = fmaf((float)((u >> 8) & 0xFF), x.y, s);
    s = fmaf((float)((u >> 16) & 0xFF), x.z, s);
    s = fmaf((float)(u >> 24), x.w, s);
    return s;
}

template <int R>
__device__ __forceinline__ void q80_step(const Q80Loads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, float (&acc)[R]) {
    float sa[R], sb[R];
#pragma unroll
    for (int r = 0; r < R; r++) sa[r] = sb[r] = 0.f;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        float4 xa[4], xb[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xa[j] = xs[(s * 16 + 4 * half + j) * kXPitch + lane];
            xb[j] = xs[(s * 16 + 8 + 4 * half + j) * kXPitch + lane];
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t w[17];
#pragma unroll
            for (int i = 0; i < 16; i++) w[i] = L[r].w[i >> 2][i & 3];
            w[16] = L[r].w16;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = 4 * half + j;
                sa[r] = q80_dot_dword(__builtin_amdgcn_alignbyte(w[i + 1], w[i], 2), xa[j], sa[r]);
                sb[r] = q80_dot_dword(w[9 + i], xb[j], sb[r]);
            }
        }
    }
    const float2 sx = reinterpret_cast<const float2*>(ss)[s * 64 + lane];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t w0 = L[r].w[0].x, w8 = L[r].w[2].x;
        const float d0 = h2f_bits(w0 & 0xFFFF), d1 = h2f_bits(w8 >> 16);
        const float v = fmaf(d0, sa[r] - sx.x, d1 * (sb[r] - sx.y));
        acc[r] += L[r].ok ? v : 0.f;
    }
}

template <int STEPS, int R>
__global__ __launch_bounds__(512) void matvec_q80_pairs_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                               float* __restrict__ y, int n_rows, int npairs) {
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + STEPS * 16 * kXPitch);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = (blockIdx.x * 8 + wave) * R;
    const int n4 = npairs * 16;  // float4 count of x
    constexpr int J = 2 * STEPS;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, 512, st);

    float acc[R];
    const uint8_t* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        rp[r] = w + (size_t)min(row0 + r, n_rows - 1) * npairs * 68;
    }
    Q80Loads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int pr = s * 64 + lane;
        const size_t off = (size_t)(min(pr, npairs - 1) + tie) * 68;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const u32x4_a4* bp = reinterpret_cast<const u32x4_a4*>(rp[r] + off);
#pragma unroll
            for (int i = 0; i < 4; i++) L[s][r].w[i] = bp[i];
            L[s][r].w16 = *reinterpret_cast<const uint32_t*>(rp[r] + off + 64);
            L[s][r].ok = row_ok[r] && pr < npairs;
        }
    };
    issue(0, 0);
    q4k_stage_store<J, false>(st, n4, tid, 512, xs, ss);
    __syncthreads();
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        q80_step<R>(L[s], xs, ss, s, lane + tie, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// Q8_K (292 bytes per 256: f32 d @0, int8 qs[256] @4, int16 sums of sixteen @260, unused here; 4-byte aligned) on the
// same scheme with the Q4_K lane map: lane (b, p) = (lane / 4, lane % 4) of a step owns the 64 quants 64p .. 64p + 63
// of superblock b -- four 16-byte loads -- and its 64 consecutive activations; d is one more dword.
struct Q8kLoads {
    u32x4 w[4];
    float d;
    bool ok;
};

template <int R>
__device__ __forceinline__ void q8k_step(const Q8kLoads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, float (&acc)[R]) {
    float sa[R];
#pragma unroll
    for (int r = 0; r < R; r++) sa[r] = 0.f;
#pragma unroll
    for (int q = 0; q < 4; q++) {  // sixteen quants at a time: one of the lane's four vectors
        float4 xv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) xv[j] = xs[(s * 16 + 4 * q + j) * kXPitch + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int j = 0; j < 4; j++) sa[r] = q80_dot_dword(L[r].w[q][j], xv[j], sa[r]);
        }
    }
    const float2 sx = reinterpret_cast<const float2*>(ss)[s * 64 + lane];  // 128 * the sums of x over the two halves
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] += L[r].ok ? L[r].d * (sa[r] - (sx.x + sx.y)) : 0.f;
}

template <int STEPS, int R>
__global__ __launch_bounds__(512) void matvec_q8k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                         float* __restrict__ y, int n_rows, int nb) {
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + STEPS * 16 * kXPitch);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 2, p = lane & 3;
    const int row0 = (blockIdx.x * 8 + wave) * R;
    const int n4 = nb * 64;  // float4 count of x
    constexpr int J = 2 * STEPS;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, 512, st);

    float acc[R];
    const uint8_t* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        rp[r] = w + (size_t)min(row0 + r, n_rows - 1) * nb * 292;
    }
    Q8kLoads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
        const size_t off = (size_t)(min(blk, nb - 1) + tie) * 292;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const u32x4_a4* bp = reinterpret_cast<const u32x4_a4*>(rp[r] + off + 4 + 64 * p);
#pragma unroll
            for (int i = 0; i < 4; i++) L[s][r].w[i] = bp[i];
            L[s][r].d = *reinterpret_cast<const float*>(rp[r] + off);
            L[s][r].ok = row_ok[r] && blk < nb;
        }
    };
    issue(0, 0);
    q4k_stage_store<J, false>(st, n4, tid, 512, xs, ss);
    __syncthreads();
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        q8k_step<R>(L[s], xs, ss, s, lane + tie, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// General form (any alignment, any block count): one wavefront per row; lane l takes blocks l, l+64, ...  The
// lane's 34 bytes are fetched as seventeen 16-bit loads (consecutive lanes read consecutive blocks, so the
// wavefront still walks one contiguous range) and x as eight aligned float4.
__global__ __launch_bounds__(256) void matvec_q8_0_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const uint8_t* rowp = w + (size_t)row * nb * 34;
    float acc = 0.f;
    for (int blk = lane; blk < nb; blk += 64) {
        const uint16_t* b16 = reinterpret_cast<const uint16_t*>(rowp + (size_t)blk * 34);
        const float d = h2f_bits(b16[0]);
        const float4* xp = reinterpret_cast<const float4*>(x + 32 * blk);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t q = (uint32_t)b16[1 + 2 * i] | ((uint32_t)b16[2 + 2 * i] << 16);
            const float4 xv = xp[i];
            s = fmaf((float)(int8_t)(q & 0xFF), xv.x, s);
            s = fmaf((float)(int8_t)((q >> 8) & 0xFF), xv.y, s);
            s = fmaf((float)(int8_t)((q >> 16) & 0xFF), xv.z, s);
            s = fmaf((float)(int8_t)(q >> 24), xv.w, s);
        }
        acc = fmaf(d, s, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

// ------------------------------------------------------------------------------------------ Q6_K
//
// 210-byte superblocks (ql[128], qh[64], int8 scales[16], f16 d), 2-byte aligned.  Main kernel (k <= 16384):
// the Q4_K scheme with four lanes per superblock.  Lane (b, j) = (lane / 4, lane % 4) of a step owns half
// n = j / 2 of superblock b and the byte positions l = 16 * (j % 2) .. + 15 in it: 16 bytes of ql[64n + l],
// 16 of ql[64n + 32 + l], 16 of qh[32n + l] -- three 128-bit loads at 2-byte alignment (the device takes
// unaligned vector loads) -- plus the eight scales of the half and d.  Those bytes hold the 64 weights
// 128n + 32q + l (q = 0..3), i.e. four runs of sixteen consecutive activations, each run under one scale.
// Four bytes at a time: the 6-bit values of run q are assembled in place,
//     (ql & 0x0F0F0F0F | qh << 4 & 0x30303030), (ql' & ... | qh << 2 & ...), (ql >> 4 & ... | qh & ...), ...
// and a byte pair masked out (v & 0x00FF00FF) is a pair of fp16 subnormals u * 2^-24 that v_fma_mix_f32
// multiplies with the fp32 activation: about 2.4 VALU operations per weight.  The zero point 32 comes back out
// as 32 * sum(x of the run), formed while x is staged; x is staged in lane order (slot 4q + i of a lane = i-th
// float4 of its run q) so the LDS reads are conflict-free and serve both rows of the wavefront.
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));

struct Q6kLoads {
    u32x4 la, lb, h;
    u32x2 sc;
    uint32_t d;
    bool ok;
};

// float4 f of x -> (step, lane, slot) of the Q6_K lane order; also the run sums, times ZERO * 2^-24 (ZERO: the quant
// that stands for zero -- 32 for Q6_K, 4 for Q3_K; 1 where the sums serve a separate minimum term, as in Q2_K)
template <int ZERO = 32>
__device__ __forceinline__ void q6k_stage_store_one(const float4& v, int f, float4* xs, float* ss) {
    const int e = 4 * f;
    const int b = e >> 8, r = e & 255;
    const int n = r >> 7, q = (r >> 5) & 3, l = r & 31;
    const int lane_all = 4 * b + 2 * n + (l >> 4);
    const int step = lane_all >> 6, ln = lane_all & 63;
    const int slot = 4 * q + ((l & 15) >> 2);
    xs[(step * 16 + slot) * kXPitch + ln] = v;
    float sum = (v.x + v.y) + (v.z + v.w);
    sum += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sum), 0xB1, 0xF, 0xF, true));  // lane ^ 1
    sum += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sum), 0x4E, 0xF, 0xF, true));  // lane ^ 2
    if ((f & 3) == 0) ss[(step * 64 + ln) * 4 + q] = sum * ((float)ZERO * 5.9604644775390625e-08f);  // ZERO * 2^-24
}

__device__ __forceinline__ float q6k_dot4(uint32_t v, const float4& x, float s) {
    const half2_t b02 = __builtin_bit_cast(half2_t, v & 0x00FF00FFu);
    const half2_t b13 = __builtin_bit_cast(half2_t, (v >> 8) & 0x00FF00FFu);
    s = fmaf((float)b02.x, x.x, s);
    s = fmaf((float)b13.x, x.y, s);
    s = fmaf((float)b02.y, x.z, s);
    s = fmaf((float)b13.y, x.w, s);
    return s;
}

template <int R>
__device__ __forceinline__ void q6k_step(const Q6kLoads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, int hsel, float (&acc)[R]) {
    float S[R][4];
#pragma unroll
    for (int r = 0; r < R; r++) S[r][0] = S[r][1] = S[r][2] = S[r][3] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 xq[4];
#pragma unroll
        for (int q = 0; q < 4; q++) xq[q] = xs[(s * 16 + 4 * q + i) * kXPitch + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t la = L[r].la[i], lb = L[r].lb[i], h = L[r].h[i];
            const uint32_t v0 = (la & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u);
            const uint32_t v1 = (lb & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u);
            const uint32_t v2 = ((la >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u);
            const uint32_t v3 = ((lb >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u);
            S[r][0] = q6k_dot4(v0, xq[0], S[r][0]);
            S[r][1] = q6k_dot4(v1, xq[1], S[r][1]);
            S[r][2] = q6k_dot4(v2, xq[2], S[r][2]);
            S[r][3] = q6k_dot4(v3, xq[3], S[r][3]);
        }
    }
    const float4 sx = reinterpret_cast<const float4*>(ss)[s * 64 + lane];
#pragma unroll
    for (int r = 0; r < R; r++) {
        // scales hsel, hsel + 2, hsel + 4, hsel + 6 of the half's eight
        const uint32_t w0 = L[r].sc.x >> (8 * hsel), w1 = L[r].sc.y >> (8 * hsel);
        const float c0 = (float)(int)(int8_t)(w0 & 0xFF), c1 = (float)(int)(int8_t)((w0 >> 16) & 0xFF);
        const float c2 = (float)(int)(int8_t)(w1 & 0xFF), c3 = (float)(int)(int8_t)((w1 >> 16) & 0xFF);
        float v = c0 * (S[r][0] - sx.x);
        v = fmaf(c1, S[r][1] - sx.y, v);
        v = fmaf(c2, S[r][2] - sx.z, v);
        v = fmaf(c3, S[r][3] - sx.w, v);
        acc[r] += L[r].ok ? h2f_bits(L[r].d) * v : 0.f;
    }
}

template <int STEPS, int R>
__global__ __launch_bounds__(512) void matvec_q6k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                         float* __restrict__ y, int n_rows, int nb) {
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + STEPS * 16 * kXPitch);  // float4 per (step, lane)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 2, j = lane & 3, n = j >> 1, hsel = j & 1;
    const int row0 = (blockIdx.x * 8 + wave) * R;
    const int n4 = nb * 64;
    constexpr int J = 2 * STEPS;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, 512, st);

    float acc[R];
    const uint8_t* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        rp[r] = w + (size_t)min(row0 + r, n_rows - 1) * nb * 210;
    }
    Q6kLoads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
        const size_t off = (size_t)(min(blk, nb - 1) + tie) * 210;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t* bp = rp[r] + off;
            L[s][r].la = *reinterpret_cast<const u32x4_a2*>(bp + 64 * n + 16 * hsel);
            L[s][r].lb = *reinterpret_cast<const u32x4_a2*>(bp + 64 * n + 32 + 16 * hsel);
            L[s][r].h = *reinterpret_cast<const u32x4_a2*>(bp + 128 + 32 * n + 16 * hsel);
            L[s][r].sc = *reinterpret_cast<const u32x2_a2*>(bp + 192 + 8 * n);
            L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 208);
            L[s][r].ok = row_ok[r] && blk < nb;
        }
    };
    issue(0, 0);
#pragma unroll
    for (int jj = 0; jj < J; jj++) {
        // a float4 index past the end repeats the last one: same data to the same slot
        const int f = min(tid + jj * 512, n4 - 1);
        q6k_stage_store_one(st.v[jj], f, xs, ss);
    }
    __syncthreads();
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        q6k_step<R>(L[s], xs, ss, s, lane + tie, hsel, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]) * 16777216.0f;
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// General form (any k): one wavefront per row, one superblock per step: lane (n, l) =
// (lane / 32, lane % 32) owns the four elements 128n + l + {0, 32, 64, 96}, which share the bytes
// ql[64n + l], ql[64n + l + 32] and qh[32n + l]; the 64 lanes read 64 consecutive bytes per load.
__global__ __launch_bounds__(256) void matvec_q6_k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const uint8_t* rowp = w + (size_t)row * nb * 210;
    const int n = lane >> 5, l = lane & 31;
    float acc = 0.f;
    for (int blk = 0; blk < nb; blk++) {
        const uint8_t* b = rowp + (size_t)blk * 210;
        const uint32_t la = b[64 * n + l], lb = b[64 * n + l + 32], h = b[128 + 32 * n + l];
        const int8_t* sc = reinterpret_cast<const int8_t*>(b + 192 + 8 * n + (l >> 4));
        const float d = h2f_bits(load_u16_a2(b + 208));
        const float* xp = x + 256 * blk + 128 * n + l;
        const float q1 = (float)((int)((la & 0xF) | ((h & 3) << 4)) - 32);
        const float q2 = (float)((int)((lb & 0xF) | (((h >> 2) & 3) << 4)) - 32);
        const float q3 = (float)((int)((la >> 4) | (((h >> 4) & 3) << 4)) - 32);
        const float q4 = (float)((int)((lb >> 4) | (((h >> 6) & 3) << 4)) - 32);
        float s = (float)sc[0] * q1 * xp[0];
        s = fmaf((float)sc[2] * q2, xp[32], s);
        s = fmaf((float)sc[4] * q3, xp[64], s);
        s = fmaf((float)sc[6] * q4, xp[96], s);
        acc = fmaf(d, s, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) y[row] = acc;
}

// ------------------------------------------------------------------------------------------ Q2_K, Q3_K
//
// The two-bit formats pack their superblock as Q6_K packs its low bits: byte qs[32n + l] holds, at bit pairs
// j = 0..3, the elements 128n + 32j + l, and the scale of an element is the one of its run of sixteen
// (8n + 2j + (l >= 16)).  So the Q6_K lane map carries over -- lane (b, jj) = (lane / 4, lane % 4) owns half
// n = jj / 2, bytes l = 16 (jj % 2) .. + 15: sixteen bytes of qs = 64 weights = four runs of sixteen consecutive
// activations under one scale each -- and with it the staging of x in lane order, the run sums, the one-step
// lookahead and the reduction.
//   Q2_K (84 bytes: scales[16], qs[64], f16 d, f16 dmin; 4-byte aligned): one 16-byte load of qs, the eight scale
//     bytes of the half, the dword d | dmin.  y = d * sum_j sc_j * (q . x)_j - dmin * sum_j m_j * (sum x)_j.
//   Q3_K (110 bytes: hmask[32], qs[64], scales[12], f16 d; 2-byte aligned): 16 bytes of qs, the 16 bytes of hmask
//     at the same l (bit 4n + j of hmask[l] is the third bit of element 128n + 32j + l), the twelve scale bytes and
//     d.  The three-bit value q | hbit << 2 stands for q - 4 + 4 hbit, so the zero point returns as 4 * sum(x of
//     the run).  Scale of run j (index is = 8n + 2j + hsel): low four bits in nibble n of byte 2j + hsel, two more
//     in bits 4n + 2 (j / 2) of byte 8 + (2j + hsel) % 4, stored with an offset of 32.
//   TQ2_0 (66 bytes: qs[64], f16 d; 2-byte aligned; ternary): the packing of Q2_K's qs with one scale, y = d (q - 1):
//     sixteen bytes of qs and d; the zero point returns as 1 * sum(x of the run).
// A byte of two or three bits masked out in pairs (v & 0x00FF00FF) is a pair of fp16 subnormals, as in Q6_K.
constexpr int kRunsQ2K = 0, kRunsQ3K = 1, kRunsTQ2 = 2;
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x3_a2 __attribute__((ext_vector_type(3), aligned(2)));

struct Q2kLoads {
    u32x4 q;
    u32x2 sc;
    uint32_t dd;
    bool ok;
};

struct Q3kLoads {
    u32x4 q, hm;
    u32x3 sc;
    uint32_t d;
    bool ok;
};

template <int R>
__device__ __forceinline__ void q2k_step(const Q2kLoads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, int hsel, float (&acc)[R]) {
    float S[R][4];
#pragma unroll
    for (int r = 0; r < R; r++) S[r][0] = S[r][1] = S[r][2] = S[r][3] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 xq[4];
#pragma unroll
        for (int q = 0; q < 4; q++) xq[q] = xs[(s * 16 + 4 * q + i) * kXPitch + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t dw = L[r].q[i];
            S[r][0] = q6k_dot4(dw & 0x03030303u, xq[0], S[r][0]);
            S[r][1] = q6k_dot4((dw >> 2) & 0x03030303u, xq[1], S[r][1]);
            S[r][2] = q6k_dot4((dw >> 4) & 0x03030303u, xq[2], S[r][2]);
            S[r][3] = q6k_dot4((dw >> 6) & 0x03030303u, xq[3], S[r][3]);
        }
    }
    const float4 sx = reinterpret_cast<const float4*>(ss)[s * 64 + lane];  // sums of x over the four runs (x 2^-24)
#pragma unroll
    for (int r = 0; r < R; r++) {
        // scale bytes hsel, hsel + 2, hsel + 4, hsel + 6 of the half's eight: low nibble scale, high nibble minimum
        const uint32_t w0 = L[r].sc.x >> (8 * hsel), w1 = L[r].sc.y >> (8 * hsel);
        float v = (float)(w0 & 0xF) * S[r][0];
        v = fmaf((float)((w0 >> 16) & 0xF), S[r][1], v);
        v = fmaf((float)(w1 & 0xF), S[r][2], v);
        v = fmaf((float)((w1 >> 16) & 0xF), S[r][3], v);
        float m = (float)((w0 >> 4) & 0xF) * sx.x;
        m = fmaf((float)((w0 >> 20) & 0xF), sx.y, m);
        m = fmaf((float)((w1 >> 4) & 0xF), sx.z, m);
        m = fmaf((float)((w1 >> 20) & 0xF), sx.w, m);
        const uint32_t dd = L[r].dd;
        const float t = fmaf(h2f_bits(dd & 0xFFFF), v, -(h2f_bits(dd >> 16) * m));
        acc[r] += L[r].ok ? t : 0.f;
    }
}

struct Tq2Loads {
    u32x4 q;
    uint32_t d;
    bool ok;
};

template <int R>
__device__ __forceinline__ void tq2_step(const Tq2Loads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, float (&acc)[R]) {
    float S[R];
#pragma unroll
    for (int r = 0; r < R; r++) S[r] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 xq[4];
#pragma unroll
        for (int q = 0; q < 4; q++) xq[q] = xs[(s * 16 + 4 * q + i) * kXPitch + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t dw = L[r].q[i];
            S[r] = q6k_dot4(dw & 0x03030303u, xq[0], S[r]);
            S[r] = q6k_dot4((dw >> 2) & 0x03030303u, xq[1], S[r]);
            S[r] = q6k_dot4((dw >> 4) & 0x03030303u, xq[2], S[r]);
            S[r] = q6k_dot4((dw >> 6) & 0x03030303u, xq[3], S[r]);
        }
    }
    const float4 sx = reinterpret_cast<const float4*>(ss)[s * 64 + lane];  // 2^-24 * sums of x over the four runs
    const float zero = (sx.x + sx.y) + (sx.z + sx.w);
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] += L[r].ok ? h2f_bits(L[r].d) * (S[r] - zero) : 0.f;
}

template <int R>
__device__ __forceinline__ void q3k_step(const Q3kLoads (&L)[R], const float4* __restrict__ xs, const float* __restrict__ ss,
                                         int s, int lane, int n, int hsel, float (&acc)[R]) {
    float S[R][4];
#pragma unroll
    for (int r = 0; r < R; r++) S[r][0] = S[r][1] = S[r][2] = S[r][3] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float4 xq[4];
#pragma unroll
        for (int q = 0; q < 4; q++) xq[q] = xs[(s * 16 + 4 * q + i) * kXPitch + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t dw = L[r].q[i], hb = L[r].hm[i] >> (4 * n);  // third bits of the half: bit j of each byte
            S[r][0] = q6k_dot4((dw & 0x03030303u) | ((hb << 2) & 0x04040404u), xq[0], S[r][0]);
            S[r][1] = q6k_dot4(((dw >> 2) & 0x03030303u) | ((hb << 1) & 0x04040404u), xq[1], S[r][1]);
            S[r][2] = q6k_dot4(((dw >> 4) & 0x03030303u) | (hb & 0x04040404u), xq[2], S[r][2]);
            S[r][3] = q6k_dot4(((dw >> 6) & 0x03030303u) | ((hb >> 1) & 0x04040404u), xq[3], S[r][3]);
        }
    }
    const float4 sx = reinterpret_cast<const float4*>(ss)[s * 64 + lane];  // 4 * 2^-24 * sums of x over the runs
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t w0 = L[r].sc.x >> (8 * hsel), w1 = L[r].sc.y >> (8 * hsel), w2 = L[r].sc.z >> (8 * hsel);
        const int lo = 4 * n;
        const float c0 = (float)((int)(((w0 >> lo) & 0xF) | (((w2 >> lo) & 3) << 4)) - 32);
        const float c1 = (float)((int)(((w0 >> (16 + lo)) & 0xF) | (((w2 >> (16 + lo)) & 3) << 4)) - 32);
        const float c2 = (float)((int)(((w1 >> lo) & 0xF) | (((w2 >> (lo + 2)) & 3) << 4)) - 32);
        const float c3 = (float)((int)(((w1 >> (16 + lo)) & 0xF) | (((w2 >> (18 + lo)) & 3) << 4)) - 32);
        float v = c0 * (S[r][0] - sx.x);
        v = fmaf(c1, S[r][1] - sx.y, v);
        v = fmaf(c2, S[r][2] - sx.z, v);
        v = fmaf(c3, S[r][3] - sx.w, v);
        acc[r] += L[r].ok ? h2f_bits(L[r].d) * v : 0.f;
    }
}

template <int STEPS, int R, int F>
__global__ __launch_bounds__(512) void matvec_runs_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                          float* __restrict__ y, int n_rows, int nb) {
    constexpr bool Q2 = F == kRunsQ2K, T2 = F == kRunsTQ2;
    constexpr int kBlock = Q2 ? 84 : T2 ? 66 : 110;
    using Loads = std::conditional_t<Q2, Q2kLoads, std::conditional_t<T2, Tq2Loads, Q3kLoads>>;
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + STEPS * 16 * kXPitch);  // float4 per (step, lane)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 2, j = lane & 3, n = j >> 1, hsel = j & 1;
    const int row0 = (blockIdx.x * 8 + wave) * R;
    const int n4 = nb * 64;
    constexpr int J = 2 * STEPS;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, 512, st);

    float acc[R];
    const uint8_t* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        rp[r] = w + (size_t)min(row0 + r, n_rows - 1) * nb * kBlock;
    }
    Loads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
        const size_t off = (size_t)(min(blk, nb - 1) + tie) * kBlock;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t* bp = rp[r] + off;
            if constexpr (Q2) {
                L[s][r].q = *reinterpret_cast<const u32x4_a4*>(bp + 16 + 32 * n + 16 * hsel);
                L[s][r].sc = *reinterpret_cast<const u32x2_a4*>(bp + 8 * n);
                L[s][r].dd = *reinterpret_cast<const uint32_t*>(bp + 80);
            } else if constexpr (T2) {
                L[s][r].q = *reinterpret_cast<const u32x4_a2*>(bp + 32 * n + 16 * hsel);
                L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 64);
            } else {
                L[s][r].q = *reinterpret_cast<const u32x4_a2*>(bp + 32 + 32 * n + 16 * hsel);
                L[s][r].hm = *reinterpret_cast<const u32x4_a2*>(bp + 16 * hsel);
                L[s][r].sc = *reinterpret_cast<const u32x3_a2*>(bp + 96);
                L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 108);
            }
            L[s][r].ok = row_ok[r] && blk < nb;
        }
    };
    issue(0, 0);
#pragma unroll
    for (int jj = 0; jj < J; jj++) {
        // a float4 index past the end repeats the last one: same data to the same slot
        const int f = min(tid + jj * 512, n4 - 1);
        q6k_stage_store_one<(Q2 || T2) ? 1 : 4>(st.v[jj], f, xs, ss);
    }
    __syncthreads();
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        if constexpr (Q2) q2k_step<R>(L[s], xs, ss, s, lane + tie, hsel, acc);
        else if constexpr (T2) tq2_step<R>(L[s], xs, ss, s, lane + tie, acc);
        else q3k_step<R>(L[s], xs, ss, s, lane + tie, n, hsel, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]) * 16777216.0f;
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// TQ1_0 (54 bytes per 256: qs u8[48] @0, qh u8[4] @48, f16 d @52; blocks 2-byte aligned).  A byte packs five trits, a qh
// byte four: trit n = ((byte * 3^n mod 256) * 3) >> 8, y = d (t - 1).  Lane (b, jj) = (lane / 4, lane % 4) of a step owns,
// of superblock b, bytes 8 jj .. 8 jj + 7 (elements 32 n + 8 jj + 0..7 for n < 5), bytes 32 + 4 jj .. + 3 (elements
// 160 + 16 n + 4 jj + 0..3) and qh byte jj (elements 240 + 4 n + jj for n < 4): 64 elements from 13 bytes.  x is staged in
// that order -- slot 2 n + h of a lane: the h-th four of its eight elements under trit n; slot 10 + n: its four of the
// second region; slot 15: its four of the third -- so a step reads sixteen float4 per lane without bank conflicts.
// Two bytes are decoded at a time in the halves of a dword: (b0 | b2 << 16) * 3^n stays inside its halves
// (255 * 81 < 2^16), so does the product with 3 after the mask, and the two trits are bytes 1 and 3 of the result
// (v_cvt_f32_ubyte1 / 3): 3.5 vector instructions per weight, the "- 1" comes back out as the sum of the lane's x.
typedef uint32_t u32_a2 __attribute__((aligned(2)));

struct Tq1Loads {
    u32x2 qa;      // bytes 8 jj .. 8 jj + 7
    uint32_t qb;   // bytes 32 + 4 jj .. + 3
    uint32_t qh;   // qh byte jj
    uint32_t d;    // f16 bits
    bool ok;
};

__device__ __forceinline__ void tq1_stage_store_one(const float4& v, int f, float4* xs) {
    const int blk = f >> 6, w = f & 63;
    const int step = blk >> 4, ln4 = (blk & 15) * 4;
    if (w < 40) {
        const int n = w >> 3, jj = (w & 7) >> 1, h = w & 1;
        xs[(step * 16 + 2 * n + h) * kXPitch + ln4 + jj] = v;
    } else if (w < 60) {
        const int n = (w - 40) >> 2, jj = (w - 40) & 3;
        xs[(step * 16 + 10 + n) * kXPitch + ln4 + jj] = v;
    } else {
        // elements 240 + 4 n + jj: component jj of this float4 is element n of lane jj's last slot
        float* last = reinterpret_cast<float*>(xs + (step * 16 + 15) * kXPitch + ln4) + (w - 60);
        last[0] = v.x, last[4] = v.y, last[8] = v.z, last[12] = v.w;
    }
}

// sum over the four bytes of q (as trit n) times the four components of x
template <int N>
__device__ __forceinline__ float tq1_dot_dword(uint32_t lo, uint32_t hi, const float4& x, float sa) {
    constexpr uint32_t kPow3 = N == 0 ? 1u : N == 1 ? 3u : N == 2 ? 9u : N == 3 ? 27u : 81u;
    const uint32_t tl = N == 0 ? lo : __umul24(lo, kPow3) & 0x00FF00FFu;
    const uint32_t th = N == 0 ? hi : __umul24(hi, kPow3) & 0x00FF00FFu;
    const uint32_t ml = __umul24(tl, 3u), mh = __umul24(th, 3u);
    sa = fmaf((float)((ml >> 8) & 0xFFu), x.x, sa);
    sa = fmaf((float)((mh >> 8) & 0xFFu), x.y, sa);
    sa = fmaf((float)(ml >> 24), x.z, sa);
    sa = fmaf((float)(mh >> 24), x.w, sa);
    return sa;
}

template <int R>
__device__ __forceinline__ void tq1_step(const Tq1Loads (&L)[R], const float4* __restrict__ xs, int s, int lane, float (&acc)[R]) {
    float4 xv[16];
    float sx = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        xv[i] = xs[(s * 16 + i) * kXPitch + lane];
        sx += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float sa = 0.f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t q = L[r].qa[h], lo = q & 0x00FF00FFu, hi = (q >> 8) & 0x00FF00FFu;
            sa = tq1_dot_dword<0>(lo, hi, xv[0 + h], sa);
            sa = tq1_dot_dword<1>(lo, hi, xv[2 + h], sa);
            sa = tq1_dot_dword<2>(lo, hi, xv[4 + h], sa);
            sa = tq1_dot_dword<3>(lo, hi, xv[6 + h], sa);
            sa = tq1_dot_dword<4>(lo, hi, xv[8 + h], sa);
        }
        {
            const uint32_t q = L[r].qb, lo = q & 0x00FF00FFu, hi = (q >> 8) & 0x00FF00FFu;
            sa = tq1_dot_dword<0>(lo, hi, xv[10], sa);
            sa = tq1_dot_dword<1>(lo, hi, xv[11], sa);
            sa = tq1_dot_dword<2>(lo, hi, xv[12], sa);
            sa = tq1_dot_dword<3>(lo, hi, xv[13], sa);
            sa = tq1_dot_dword<4>(lo, hi, xv[14], sa);
        }
        {
            // the qh byte: trits 0..3 against the four components of the last slot
            const uint32_t b = L[r].qh;
            const uint32_t t01 = (b | (__umul24(b, 3u) << 16)) & 0x00FF00FFu;      // b, 3 b mod 256
            const uint32_t t23 = (__umul24(b, 9u) & 0xFFu) | ((__umul24(b, 27u) & 0xFFu) << 16);
            const uint32_t m01 = __umul24(t01, 3u), m23 = __umul24(t23, 3u);
            sa = fmaf((float)((m01 >> 8) & 0xFFu), xv[15].x, sa);
            sa = fmaf((float)(m01 >> 24), xv[15].y, sa);
            sa = fmaf((float)((m23 >> 8) & 0xFFu), xv[15].z, sa);
            sa = fmaf((float)(m23 >> 24), xv[15].w, sa);
        }
        acc[r] += L[r].ok ? h2f_bits((uint16_t)L[r].d) * (sa - sx) : 0.f;
    }
}

template <int STEPS, int R>
__global__ __launch_bounds__(512) void matvec_tq1_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                         float* __restrict__ y, int n_rows, int nb) {
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 2, jj = lane & 3;
    const int row0 = (blockIdx.x * 8 + wave) * R;
    const int n4 = nb * 64;  // float4 count of x
    constexpr int J = 2 * STEPS;
    Q4kStage<J> st;
    q4k_stage_load<J>(x, n4, tid, 512, st);

    float acc[R];
    const uint8_t* rp[R];
    bool row_ok[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = 0.f;
        row_ok[r] = row0 + r < n_rows;
        rp[r] = w + (size_t)min(row0 + r, n_rows - 1) * nb * 54;
    }
    Tq1Loads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
        const size_t off = (size_t)(min(blk, nb - 1) + tie) * 54;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t* bp = rp[r] + off;
            L[s][r].qa = *reinterpret_cast<const u32x2_a2*>(bp + 8 * jj);
            L[s][r].qb = *reinterpret_cast<const u32_a2*>(bp + 32 + 4 * jj);
            L[s][r].qh = bp[48 + jj];
            L[s][r].d = load_u16_a2(bp + 52);
            L[s][r].ok = row_ok[r] && blk < nb;
        }
    };
    issue(0, 0);
#pragma unroll
    for (int j = 0; j < J; j++) tq1_stage_store_one(st.v[j], min(tid + j * 512, n4 - 1), xs);
    __syncthreads();
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        tq1_step<R>(L[s], xs, s, lane + tie, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float total = wave_sum(acc[r]);
        if (lane == 0 && row_ok[r]) y[row0 + r] = total;
    }
}

// What the rotary epilogue needs beyond the row totals, formed at the top of the kernel so that its dependent
// loads (position, then page id) and the sine / cosine are off the tail of the wavefront.
struct Q4kRopeCtx {
    int which = 0, h = 0, e = 0, page = 0, slot = 0;  // q / k / v, head, element pair, cache page and slot
    float sn = 0.f, cs = 1.f;
};

// element index (even) inside its head of the rotary pair that output unit `unit` holds
__device__ __forceinline__ int q4k_rope_elem(const skn_q4k_segments& seg, const skn_rope_epilogue& rope, int unit) {
    int row = unit * 2;
    row -= row >= seg.rows[0] + seg.rows[1] ? seg.rows[0] + seg.rows[1] : row >= seg.rows[0] ? seg.rows[0] : 0;
    return row % rope.head_dim;
}

__device__ __forceinline__ Q4kRopeCtx q4k_rope_prepare(const skn_q4k_segments& seg, const skn_rope_epilogue& rope,
                                                     int unit, int pos, int page, double freq) {
    Q4kRopeCtx c;
    int row = unit * 2;  // rows 2u, 2u+1 of the stacked q | k | v output: one rotary pair (segment sizes are even)
    c.which = row >= seg.rows[0] + seg.rows[1] ? 2 : row >= seg.rows[0] ? 1 : 0;
    row -= c.which == 2 ? seg.rows[0] + seg.rows[1] : c.which == 1 ? seg.rows[0] : 0;
    c.h = row / rope.head_dim;
    c.e = row % rope.head_dim;
    c.slot = pos % rope.page_tokens;
    c.page = page;
    if (rope.inv_freq) skn_rope_sincos_freq(pos, freq, &c.sn, &c.cs);
    else skn_rope_sincos(pos, c.e, rope.head_dim, rope.log2_base, &c.sn, &c.cs);
    return c;
}

// What the first lane does with the two row totals of unit `unit` (rows 2*unit, 2*unit + 1; for SwiGLU: row
// `unit` of gate and of up).
template <int EPI>
__device__ __forceinline__ void q4k_epilogue(const skn_rope_epilogue& rope, const Q4kRopeCtx& rc,
                                             float* __restrict__ y, int n_out, int unit, float t0, float t1) {
    const bool ok0 = EPI == SKN_EPI_SWIGLU ? unit < n_out : 2 * unit < n_out;
    const bool ok1 = EPI == SKN_EPI_SWIGLU ? ok0 : 2 * unit + 1 < n_out;
    if (EPI == SKN_EPI_ROPE) {
        if (ok0) {
            float a = t0, b = t1;
            if (rc.which < 2) {
                a = t0 * rc.cs - t1 * rc.sn;
                b = t0 * rc.sn + t1 * rc.cs;
            }
            if (rc.which == 0) {
                y[rc.h * rope.head_dim + rc.e] = a;
                y[rc.h * rope.head_dim + rc.e + 1] = b;
            } else {
                const size_t dst =
                    (((size_t)rc.page * rope.n_head + rc.h) * rope.page_tokens + rc.slot) * rope.head_dim + rc.e;
                const uint32_t packed = (uint32_t)__half_as_ushort(__float2half_rn(a)) |
                                        ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
                *reinterpret_cast<uint32_t*>((rc.which == 1 ? rope.k_pool : rope.v_pool) + dst) = packed;
            }
        }
    } else if (EPI == SKN_EPI_SWIGLU) {
        if (ok0) y[unit] = t0 / (1.0f + expf(-t0)) * t1;
    } else if (EPI == SKN_EPI_ADD) {
        if (ok0) y[unit * 2] += t0;
        if (ok1) y[unit * 2 + 1] += t1;
    } else {
        if (ok0) y[unit * 2] = t0;
        if (ok1) y[unit * 2 + 1] = t1;
    }
}

// One float4 of the attention output out of the unmerged partials of S splits: sum_s w_s part_s / sum_s w_s l_s with
// w_s = exp(max_s - max over the splits); (max, sum) of split s and head h at ml[s * pairs + h].
template <int S>
__device__ __forceinline__ float4 q4k_merge_splits(const float4* __restrict__ part, const float2* __restrict__ ml, int n4, int f,
                                                   int head, int pairs) {
    float2 e[S];
    float4 v[S];
#pragma unroll
    for (int sp = 0; sp < S; sp++) e[sp] = ml[sp * pairs + head];
#pragma unroll
    for (int sp = 0; sp < S; sp++) v[sp] = part[(size_t)sp * n4 + f];
    float mx = e[0].x;
#pragma unroll
    for (int sp = 1; sp < S; sp++) mx = fmaxf(mx, e[sp].x);
    const float m_safe = mx == -INFINITY ? 0.f : mx;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    float den = 0.f;
#pragma unroll
    for (int sp = 0; sp < S; sp++) {
        const float wgt = __expf(e[sp].x - m_safe);
        a.x = fmaf(wgt, v[sp].x, a.x), a.y = fmaf(wgt, v[sp].y, a.y), a.z = fmaf(wgt, v[sp].z, a.z), a.w = fmaf(wgt, v[sp].w, a.w);
        den = fmaf(wgt, e[sp].y, den);
    }
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    return make_float4(a.x * inv, a.y * inv, a.z * inv, a.w * inv);
}

// ---- fused forms used by the decoder ---------------------------------------------------------------------
// Up to three weight matrices with the same k stacked along the output axis (q, k, v projections in one launch;
// gate and up paired row by row), optional RMSNorm of x folded into the staging (every workgroup needs all of
// x anyway, so it also forms sum(x^2) and stores x * r * norm_w), and an epilogue that stores, adds into the
// residual stream, or applies SwiGLU to a (gate, up) row pair.  Two rows per wavefront.
// F: the format of all the matrices of the launch, as in matvec_q4k_kernel.
template <int STEPS, int EPI, bool NORM, int F = kFmtQ4K>
__global__ __launch_bounds__(512) void matvec_q4k_fused_kernel(skn_q4k_segments seg, const float* __restrict__ x,
                                                               const float* __restrict__ norm_w, float eps,
                                                               float* __restrict__ y, int n_out, int nb,
                                                               skn_rope_epilogue rope) {
    constexpr int R = 2;
    constexpr bool Q5 = F == kFmtQ5K, Q6 = F == kFmtQ6K, Q8 = F == kFmtQ80, Q2 = F == kFmtQ2K, Q3 = F == kFmtQ3K, Q8K = F == kFmtQ8K;
    constexpr bool T2 = F == kFmtTQ2, T1 = F == kFmtTQ1;
    constexpr bool kRuns = Q6 || Q2 || Q3 || T2;  // the Q6_K lane map: four runs of sixteen per lane, a float4 of run sums
    constexpr bool kXS = F == kFmtIQ4XS;
    constexpr bool kSmall = F >= kFmtQ40 && F <= kFmtIQ4XS && !Q6 && !Q8;
    using Loads = std::conditional_t<Q8, Q80Loads, std::conditional_t<Q6, Q6kLoads, std::conditional_t<Q2, Q2kLoads, std::conditional_t<Q3, Q3kLoads,
                  std::conditional_t<T2, Tq2Loads, std::conditional_t<T1, Tq1Loads,
                  std::conditional_t<Q8K, Q8kLoads, std::conditional_t<kSmall, Q4xLoads, std::conditional_t<Q5, Q5kLoads, Q4kLoads>>>>>>>>>;
    constexpr int kChunks = Q5 ? 11 : 9, kFirst = Q5 ? 3 : 1;
    constexpr int kSmallBytes = (F == kFmtQ40 || F == kFmtIQ4NL) ? 18 : (F == kFmtQ41 ? 20 : (F == kFmtQ50 ? 22 : 24)), kHi = kSmall ? 4 : 8;
    constexpr bool kPlainX = F == kFmtIQ4NL || kXS;  // x staged unscaled, block sums times 128, results in true units
    extern __shared__ float4 lds4[];
    float4* xs = lds4;
    float* ss = reinterpret_cast<float*>(lds4 + STEPS * 16 * kXPitch);
    float* red = ss + STEPS * (kRuns ? 256 : 128);  // eight partial sums of x^2 (all LDS here is dynamic)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane >> 2, p = lane & 3;
    const int n4 = nb * 64;
    constexpr int J = 2 * STEPS;  // 512 threads x J float4 cover k <= STEPS * 4096

    // rotary epilogue: the position and, once it is known, the page id of its cache row are requested here (two
    // dependent round trips) so that neither is waited for after the staging barrier
    int rope_pos = 0, rope_page = 0;
    double rope_freq = 0.0;  // (the pair's frequency out of the model's table, requested with the position)
    if (EPI == SKN_EPI_ROPE) {
        rope_pos = rope.pos_dev[0];
        if (rope.inv_freq)
            rope_freq = rope.inv_freq[q4k_rope_elem(seg, rope, min((int)(blockIdx.x * 8 + (threadIdx.x >> 6)), (n_out + 1) / 2 - 1)) >> 1];
    }
    Q4kStage<J> st, nw;
    bool merged = false;
    if constexpr (EPI == SKN_EPI_ADD && !NORM) {
        // x as the unmerged split partials of the decode attention: float4 f of x belongs to head f / head_f4; its value
        // is sum_s w_s * part_s / sum_s w_s * l_s with w_s = exp(max_s - max over the splits), the merge the attention
        // kernel otherwise does behind a device-wide counter
        if (rope.merge_splits > 1) {
            merged = true;
            const float4* part = reinterpret_cast<const float4*>(x);
            const float2* ml = reinterpret_cast<const float2*>(rope.merge_ml);
#pragma unroll
            for (int j = 0; j < J; j++) {
                const int f = min(tid + j * 512, n4 - 1), head = f / rope.merge_head_f4;
                // (the split count as a constant: every load of a float4's merge is requested before any is used)
                switch (rope.merge_splits) {
                    case 2: st.v[j] = q4k_merge_splits<2>(part, ml, n4, f, head, rope.merge_pairs); break;
                    case 4: st.v[j] = q4k_merge_splits<4>(part, ml, n4, f, head, rope.merge_pairs); break;
                    default: st.v[j] = q4k_merge_splits<8>(part, ml, n4, f, head, rope.merge_pairs); break;
                }
            }
        }
    }
    if (!merged) q4k_stage_load<J>(x, n4, tid, 512, st);
    if (NORM) q4k_stage_load<J>(norm_w, n4, tid, 512, nw);

    // the two rows of this wavefront: consecutive rows of the stacked matrices, or row i of gate and of up
    const int unit = blockIdx.x * 8 + wave;
    const uint8_t* rowp[R];
    bool row_ok[R];
    const size_t row_bytes = (size_t)nb * (Q8 ? 272 : Q6 ? 210 : Q2 ? 84 : Q3 ? 110 : T2 ? 66 : T1 ? 54 : Q8K ? 292 : kXS ? 136 : kSmall ? 8 * kSmallBytes : 16 * kChunks);
    if (EPI == SKN_EPI_SWIGLU) {
        const int i = min(unit, n_out - 1);
        row_ok[0] = row_ok[1] = unit < n_out;
        rowp[0] = seg.w[0] + (size_t)i * row_bytes;
        rowp[1] = seg.w[1] + (size_t)i * row_bytes;
    } else {
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = unit * R + r;
            row_ok[r] = row < n_out;
            row = min(row, n_out - 1);
            const uint8_t* base = seg.w[0];
            if (row >= seg.rows[0]) {
                row -= seg.rows[0];
                base = seg.w[1];
                if (row >= seg.rows[1]) {
                    row -= seg.rows[1];
                    base = seg.w[2];
                }
            }
            rowp[r] = base + (size_t)row * row_bytes;
        }
    }
    Loads L[STEPS][R];
    auto issue = [&](int s, int tie) __attribute__((always_inline)) {
        const int blk = s * 16 + sub;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if constexpr (Q8) {  // lane = pair of blocks, 64 pairs per step
                const int pr = s * 64 + lane, npairs = 4 * nb;
                const uint8_t* bp = rowp[r] + (size_t)(min(pr, npairs - 1) + tie) * 68;
#pragma unroll
                for (int i = 0; i < 4; i++) L[s][r].w[i] = reinterpret_cast<const u32x4_a4*>(bp)[i];
                L[s][r].w16 = *reinterpret_cast<const uint32_t*>(bp + 64);
                L[s][r].ok = row_ok[r] && pr < npairs;
            } else if constexpr (Q6) {
                const int n = p >> 1, hsel = p & 1;
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 210;
                L[s][r].la = *reinterpret_cast<const u32x4_a2*>(bp + 64 * n + 16 * hsel);
                L[s][r].lb = *reinterpret_cast<const u32x4_a2*>(bp + 64 * n + 32 + 16 * hsel);
                L[s][r].h = *reinterpret_cast<const u32x4_a2*>(bp + 128 + 32 * n + 16 * hsel);
                L[s][r].sc = *reinterpret_cast<const u32x2_a2*>(bp + 192 + 8 * n);
                L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 208);
            } else if constexpr (Q2) {
                const int n = p >> 1, hsel = p & 1;
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 84;
                L[s][r].q = *reinterpret_cast<const u32x4_a4*>(bp + 16 + 32 * n + 16 * hsel);
                L[s][r].sc = *reinterpret_cast<const u32x2_a4*>(bp + 8 * n);
                L[s][r].dd = *reinterpret_cast<const uint32_t*>(bp + 80);
            } else if constexpr (Q3) {
                const int n = p >> 1, hsel = p & 1;
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 110;
                L[s][r].q = *reinterpret_cast<const u32x4_a2*>(bp + 32 + 32 * n + 16 * hsel);
                L[s][r].hm = *reinterpret_cast<const u32x4_a2*>(bp + 16 * hsel);
                L[s][r].sc = *reinterpret_cast<const u32x3_a2*>(bp + 96);
                L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 108);
            } else if constexpr (T2) {
                const int n = p >> 1, hsel = p & 1;
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 66;
                L[s][r].q = *reinterpret_cast<const u32x4_a2*>(bp + 32 * n + 16 * hsel);
                L[s][r].d = *reinterpret_cast<const uint16_t*>(bp + 64);
            } else if constexpr (T1) {
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 54;
                L[s][r].qa = *reinterpret_cast<const u32x2_a2*>(bp + 8 * p);
                L[s][r].qb = *reinterpret_cast<const u32_a2*>(bp + 32 + 4 * p);
                L[s][r].qh = bp[48 + p];
                L[s][r].d = load_u16_a2(bp + 52);
            } else if constexpr (Q8K) {
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) + tie) * 292;
#pragma unroll
                for (int i = 0; i < 4; i++) L[s][r].w[i] = reinterpret_cast<const u32x4_a4*>(bp + 4 + 64 * p)[i];
                L[s][r].d = *reinterpret_cast<const float*>(bp);
            } else if constexpr (kXS) {
                iq4xs_load(rowp[r] + (size_t)min(blk, nb - 1) * 136 + tie, p, L[s][r]);
            } else if constexpr (kSmall) {
                const uint8_t* bp = rowp[r] + (size_t)(min(blk, nb - 1) * 8 + 2 * p) * kSmallBytes + tie;
                q4x_load<F>(bp, L[s][r]);
            } else {
                const u32x4* bp = reinterpret_cast<const u32x4*>(rowp[r]) + min(blk, nb - 1) * kChunks + kFirst + 2 * p + tie;
                L[s][r].qa = bp[0];
                L[s][r].qb = bp[1];
                L[s][r].h = bp[-kFirst - 2 * p];
                if constexpr (Q5) {
                    L[s][r].ha = bp[1 - kFirst - 2 * p];
                    L[s][r].hb = bp[2 - kFirst - 2 * p];
                }
            }
            if constexpr (!Q8) L[s][r].ok = row_ok[r] && blk < nb;
        }
    };
    issue(0, 0);
    if (EPI == SKN_EPI_ROPE) rope_page = rope.page_table[rope_pos / rope.page_tokens];

    // RMSNorm: y = sum_k W[., k] * (x_k * r * g_k) = r * sum_k W[., k] * (x_k * g_k): x * g is staged and the row
    // totals are multiplied by r = 1 / sqrt(mean(x^2) + eps) at the end, so the sum of squares needs no
    // barrier of its own (its eight partials are read after the staging barrier)
    if (NORM) {
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < J; j++) {
            if (tid + j * 512 < n4) {
                const float4 v = st.v[j];
                sq += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
            }
            st.v[j].x *= nw.v[j].x;
            st.v[j].y *= nw.v[j].y;
            st.v[j].z *= nw.v[j].z;
            st.v[j].w *= nw.v[j].w;
        }
        sq = wave_sum(sq);
        if (lane == 0) red[wave] = sq;
    }
    if constexpr (Q8 || Q8K) {
        q4k_stage_store<J, false>(st, n4, tid, 512, xs, ss);
    } else if constexpr (kRuns) {
#pragma unroll
        for (int jj = 0; jj < J; jj++) q6k_stage_store_one<Q6 ? 32 : Q3 ? 4 : 1>(st.v[jj], min(tid + jj * 512, n4 - 1), xs, ss);
    } else if constexpr (T1) {
#pragma unroll
        for (int jj = 0; jj < J; jj++) tq1_stage_store_one(st.v[jj], min(tid + jj * 512, n4 - 1), xs);
    } else {
        q4k_stage_store<J, !kPlainX, kHi>(st, n4, tid, 512, xs, ss);
    }
    __syncthreads();
    // (after the staging, while the first weights are still on their way)
    Q4kRopeCtx rc;
    if (EPI == SKN_EPI_ROPE) rc = q4k_rope_prepare(seg, rope, min(unit, (n_out + 1) / 2 - 1), rope_pos, rope_page, rope_freq);
    float rinv = 1.0f;
    if (NORM) {
        const float total = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
        rinv = 1.0f / sqrtf(total / (float)(nb * 256) + eps);
    }

    float acc[R] = {0.f, 0.f};
    int tie = 0;
    asm volatile("" : "+v"(tie));
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        if (s + 1 < STEPS) issue(s + 1, tie);
        asm volatile("" ::: "memory");
        if constexpr (Q8) q80_step<R>(L[s], xs, ss, s, lane + tie, acc);
        else if constexpr (Q8K) q8k_step<R>(L[s], xs, ss, s, lane + tie, acc);
        else if constexpr (Q6) q6k_step<R>(L[s], xs, ss, s, lane + tie, p & 1, acc);
        else if constexpr (Q2) q2k_step<R>(L[s], xs, ss, s, lane + tie, p & 1, acc);
        else if constexpr (Q3) q3k_step<R>(L[s], xs, ss, s, lane + tie, p >> 1, p & 1, acc);
        else if constexpr (T2) tq2_step<R>(L[s], xs, ss, s, lane + tie, acc);
        else if constexpr (T1) tq1_step<R>(L[s], xs, s, lane + tie, acc);
        else if constexpr (kSmall) q4x_step<R, F>(L[s], xs, ss, s, lane + tie, acc);
        else q4k_step<R>(L[s], xs, ss, s, lane + tie, p, acc);
        asm volatile("" : "+v"(tie), "+v"(acc[R - 1]));
    }
    const float back = (Q8 || Q8K || T1 || kPlainX) ? rinv : 16777216.0f * rinv;  // (the nibble formats work in units of 2^-24)
    const float t0 = wave_sum(acc[0]) * back;
    const float t1 = wave_sum(acc[1]) * back;
    if (lane == 0) q4k_epilogue<EPI>(rope, rc, y, n_out, unit, t0, t1);
}

template <int STEPS, int EPI, bool NORM, int F>
int launch_q4k_fused(skn_ctx* ctx, const skn_q4k_segments& seg, int n_out, int nb, const float* x, const float* norm_w,
                     float eps, float* y, const skn_rope_epilogue& rope) {
    const size_t lds = (size_t)STEPS * (16 * kXPitch * sizeof(float4) + 64 * ((F == kFmtQ6K || F == kFmtQ2K || F == kFmtQ3K || F == kFmtTQ2) ? sizeof(float4) : sizeof(float2))) + 8 * sizeof(float);
    const int units = EPI == SKN_EPI_SWIGLU ? n_out : (n_out + 1) / 2;
    dim3 grid((unsigned)((units + 7) / 8)), block(512);
    skn_launch(ctx, matvec_q4k_fused_kernel<STEPS, EPI, NORM, F>, grid, block, lds, seg, x, norm_w, eps, y, n_out, nb, rope);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int STEPS, int F>
int dispatch_q4k_fused(skn_ctx* ctx, const skn_q4k_segments& seg, int n_out, int nb, const float* x, const float* norm_w,
                       float eps, float* y, int epi, const skn_rope_epilogue& rope) {
    const bool norm = norm_w != nullptr;
    if (epi == SKN_EPI_ROPE)
        return norm ? launch_q4k_fused<STEPS, SKN_EPI_ROPE, true, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope)
                    : launch_q4k_fused<STEPS, SKN_EPI_ROPE, false, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope);
    if (epi == SKN_EPI_SWIGLU)
        return norm ? launch_q4k_fused<STEPS, SKN_EPI_SWIGLU, true, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope)
                    : launch_q4k_fused<STEPS, SKN_EPI_SWIGLU, false, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope);
    if (epi == SKN_EPI_ADD)
        return norm ? launch_q4k_fused<STEPS, SKN_EPI_ADD, true, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope)
                    : launch_q4k_fused<STEPS, SKN_EPI_ADD, false, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope);
    return norm ? launch_q4k_fused<STEPS, SKN_EPI_STORE, true, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope)
                : launch_q4k_fused<STEPS, SKN_EPI_STORE, false, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, rope);
}

template <int STEPS, int EPI, bool NORM, int F>
hipError_t allow_big_lds_fused() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_q4k_fused_kernel<STEPS, EPI, NORM, F>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS, int F>
hipError_t allow_big_lds_fused_all() {
    hipError_t e = allow_big_lds_fused<STEPS, SKN_EPI_STORE, false, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_STORE, true, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_ADD, false, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_ADD, true, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_SWIGLU, false, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_SWIGLU, true, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_ROPE, false, F>();
    if (e == hipSuccess) e = allow_big_lds_fused<STEPS, SKN_EPI_ROPE, true, F>();
    return e;
}

template <int STEPS, int R, int F = kFmtQ4K>
int launch_q4k(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y, int waves) {
    if (STEPS > 0 && waves != 8) return launch_q4k<0, R, F>(ctx, w, n, nb, x, y, waves);
    const int steps = (nb + 15) / 16;
    const size_t lds = (size_t)steps * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float2));
    SKN_REQUIRE(ctx, lds <= 160 * 1024, SKN_ERR_SHAPE, "skn_matvec_q: k = %d needs %zu bytes of LDS (limit 163840)",
                nb * 256, lds);
    auto kern = matvec_q4k_kernel<STEPS, R, F>;
    const int rows_per_wg = waves * R;
    dim3 grid((unsigned)((n + rows_per_wg - 1) / rows_per_wg)), block((unsigned)(waves * 64));
    skn_launch(ctx, kern, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int R, int F = kFmtQ4K>
int dispatch_q4k(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y, int waves) {
    switch ((nb + 15) / 16) {
        case 1: return launch_q4k<1, R, F>(ctx, w, n, nb, x, y, waves);
        case 2: return launch_q4k<2, R, F>(ctx, w, n, nb, x, y, waves);
        case 3: return launch_q4k<3, R, F>(ctx, w, n, nb, x, y, waves);
        case 4: return launch_q4k<4, R, F>(ctx, w, n, nb, x, y, waves);
        default: return launch_q4k<0, R, F>(ctx, w, n, nb, x, y, waves);
    }
}

template <int STEPS>
int launch_q80_pairs(skn_ctx* ctx, const uint8_t* w, int n, int npairs, const float* x, float* y) {
    constexpr int R = 2;
    const size_t lds = (size_t)STEPS * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float2));
    dim3 grid((unsigned)((n + 8 * R - 1) / (8 * R))), block(512);
    skn_launch(ctx, matvec_q80_pairs_kernel<STEPS, R>, grid, block, lds, w, x, y, n, npairs);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int STEPS>
int launch_q6k(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y) {
    constexpr int R = 1;
    const size_t lds = (size_t)STEPS * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float4));
    dim3 grid((unsigned)((n + 8 * R - 1) / (8 * R))), block(512);
    skn_launch(ctx, matvec_q6k_kernel<STEPS, R>, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

// Q2_K / Q3_K on the Q6_K lane map: two rows per wavefront while a row is one or two steps, one beyond
template <int STEPS, int F>
int launch_runs(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y) {
    constexpr int R = STEPS <= 2 ? 2 : 1;
    const size_t lds = (size_t)STEPS * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float4));
    dim3 grid((unsigned)((n + 8 * R - 1) / (8 * R))), block(512);
    skn_launch(ctx, matvec_runs_kernel<STEPS, R, F>, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int F>
int dispatch_runs(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y) {
    switch ((nb + 15) / 16) {
        case 1: return launch_runs<1, F>(ctx, w, n, nb, x, y);
        case 2: return launch_runs<2, F>(ctx, w, n, nb, x, y);
        case 3: return launch_runs<3, F>(ctx, w, n, nb, x, y);
        default: return launch_runs<4, F>(ctx, w, n, nb, x, y);
    }
}

template <int STEPS, int F>
hipError_t allow_big_lds_runs() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_runs_kernel<STEPS, (STEPS <= 2 ? 2 : 1), F>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS>
int launch_q8k(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y) {
    constexpr int R = STEPS <= 2 ? 2 : 1;
    const size_t lds = (size_t)STEPS * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float2));
    dim3 grid((unsigned)((n + 8 * R - 1) / (8 * R))), block(512);
    skn_launch(ctx, matvec_q8k_kernel<STEPS, R>, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int STEPS>
int launch_tq1(skn_ctx* ctx, const uint8_t* w, int n, int nb, const float* x, float* y) {
    constexpr int R = STEPS <= 2 ? 2 : 1;
    const size_t lds = (size_t)STEPS * 16 * kXPitch * sizeof(float4);
    dim3 grid((unsigned)((n + 8 * R - 1) / (8 * R))), block(512);
    skn_launch(ctx, matvec_tq1_kernel<STEPS, R>, grid, block, lds, w, x, y, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

template <int STEPS>
hipError_t allow_big_lds_tq1() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_tq1_kernel<STEPS, (STEPS <= 2 ? 2 : 1)>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS>
hipError_t allow_big_lds_q8k() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_q8k_kernel<STEPS, (STEPS <= 2 ? 2 : 1)>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS>
hipError_t allow_big_lds_q6k() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_q6k_kernel<STEPS, 1>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS>
hipError_t allow_big_lds_q80() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_q80_pairs_kernel<STEPS, 2>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

template <int STEPS, int R, int F = kFmtQ4K>
hipError_t allow_big_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(matvec_q4k_kernel<STEPS, R, F>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}

}  // namespace

// Dynamic LDS above 48 KiB must be allowed per kernel; done once here so that no launch path (which may run under
// stream capture) has to.
int skn_matvec_init(skn_ctx* ctx) {
    hipError_t (*fns[])() = {allow_big_lds<0, 1>, allow_big_lds<1, 1>, allow_big_lds<2, 1>, allow_big_lds<3, 1>,
                             allow_big_lds<4, 1>, allow_big_lds<0, 2>, allow_big_lds<1, 2>, allow_big_lds<2, 2>,
                             allow_big_lds<3, 2>, allow_big_lds<4, 2>, allow_big_lds<0, 4>, allow_big_lds<1, 4>,
                             allow_big_lds<2, 4>, allow_big_lds<3, 4>, allow_big_lds<4, 4>,
#define SKN_ALLOW_FMT(F)                                                                                       \
    allow_big_lds<0, 1, F>, allow_big_lds<1, 1, F>, allow_big_lds<2, 1, F>, allow_big_lds<3, 1, F>,             \
        allow_big_lds<4, 1, F>, allow_big_lds<0, 2, F>, allow_big_lds<1, 2, F>, allow_big_lds<2, 2, F>,         \
        allow_big_lds<3, 2, F>, allow_big_lds<4, 2, F>
                             SKN_ALLOW_FMT(kFmtQ5K), SKN_ALLOW_FMT(kFmtQ40), SKN_ALLOW_FMT(kFmtQ41),
                             SKN_ALLOW_FMT(kFmtQ50), SKN_ALLOW_FMT(kFmtQ51), SKN_ALLOW_FMT(kFmtIQ4NL),
                             SKN_ALLOW_FMT(kFmtIQ4XS)};
#undef SKN_ALLOW_FMT
    for (auto f : fns) SKN_HIP(ctx, f());
    SKN_HIP(ctx, allow_big_lds_q6k<1>());
    SKN_HIP(ctx, allow_big_lds_q6k<2>());
    SKN_HIP(ctx, allow_big_lds_q6k<3>());
    SKN_HIP(ctx, allow_big_lds_q6k<4>());
    SKN_HIP(ctx, (allow_big_lds_runs<1, kRunsQ2K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<2, kRunsQ2K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<3, kRunsQ2K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<4, kRunsQ2K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<1, kRunsQ3K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<2, kRunsQ3K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<3, kRunsQ3K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<4, kRunsQ3K>()));
    SKN_HIP(ctx, (allow_big_lds_runs<1, kRunsTQ2>()));
    SKN_HIP(ctx, (allow_big_lds_runs<2, kRunsTQ2>()));
    SKN_HIP(ctx, (allow_big_lds_runs<3, kRunsTQ2>()));
    SKN_HIP(ctx, (allow_big_lds_runs<4, kRunsTQ2>()));
    SKN_HIP(ctx, allow_big_lds_tq1<1>());
    SKN_HIP(ctx, allow_big_lds_tq1<2>());
    SKN_HIP(ctx, allow_big_lds_tq1<3>());
    SKN_HIP(ctx, allow_big_lds_tq1<4>());
    SKN_HIP(ctx, allow_big_lds_q8k<1>());
    SKN_HIP(ctx, allow_big_lds_q8k<2>());
    SKN_HIP(ctx, allow_big_lds_q8k<3>());
    SKN_HIP(ctx, allow_big_lds_q8k<4>());
    SKN_HIP(ctx, allow_big_lds_q80<1>());
    SKN_HIP(ctx, allow_big_lds_q80<2>());
    SKN_HIP(ctx, allow_big_lds_q80<3>());
    SKN_HIP(ctx, allow_big_lds_q80<4>());
#define SKN_ALLOW_FUSED(F)                              \
    SKN_HIP(ctx, (allow_big_lds_fused_all<1, F>()));    \
    SKN_HIP(ctx, (allow_big_lds_fused_all<2, F>()));    \
    SKN_HIP(ctx, (allow_big_lds_fused_all<3, F>()));    \
    SKN_HIP(ctx, (allow_big_lds_fused_all<4, F>()))
    SKN_ALLOW_FUSED(kFmtQ4K);
    SKN_ALLOW_FUSED(kFmtQ5K);
    SKN_ALLOW_FUSED(kFmtQ40);
    SKN_ALLOW_FUSED(kFmtQ41);
    SKN_ALLOW_FUSED(kFmtQ50);
    SKN_ALLOW_FUSED(kFmtQ51);
    SKN_ALLOW_FUSED(kFmtQ6K);
    SKN_ALLOW_FUSED(kFmtQ80);
    SKN_ALLOW_FUSED(kFmtIQ4NL);
    SKN_ALLOW_FUSED(kFmtIQ4XS);
    SKN_ALLOW_FUSED(kFmtQ2K);
    SKN_ALLOW_FUSED(kFmtQ3K);
    SKN_ALLOW_FUSED(kFmtQ8K);
    SKN_ALLOW_FUSED(kFmtTQ2);
    SKN_ALLOW_FUSED(kFmtTQ1);
#undef SKN_ALLOW_FUSED
    return SKN_OK;
}

bool skn_matvec_fusable(int ggml_type) {
    return ggml_type == SKN_TYPE_Q4_K || ggml_type == SKN_TYPE_Q5_K || ggml_type == SKN_TYPE_Q4_0 ||
           ggml_type == SKN_TYPE_Q4_1 || ggml_type == SKN_TYPE_Q5_0 || ggml_type == SKN_TYPE_Q5_1 ||
           ggml_type == SKN_TYPE_Q6_K || ggml_type == SKN_TYPE_Q8_0 || ggml_type == SKN_TYPE_IQ4_NL ||
           ggml_type == SKN_TYPE_IQ4_XS || ggml_type == SKN_TYPE_Q2_K || ggml_type == SKN_TYPE_Q3_K || ggml_type == SKN_TYPE_Q8_K ||
           ggml_type == SKN_TYPE_TQ1_0 || ggml_type == SKN_TYPE_TQ2_0;
}

// Fused matvec for the decoder, all matrices of one of the formats above; k <= 16384 (four unrolled steps).
// Returns SKN_ERR_SHAPE otherwise.
int skn_matvec_q4k_fused(skn_ctx* ctx, const skn_q4k_segments& seg, int n_out, int k, const float* x, const float* norm_w,
                         float eps, float* y, int epi, const skn_rope_epilogue* rope_in, int ggml_type) {
    SKN_REQUIRE(ctx, skn_matvec_fusable(ggml_type), SKN_ERR_TYPE, "fused matvec: ggml type %d has no fused kernel", ggml_type);
    {
        const uintptr_t mask = (ggml_type == SKN_TYPE_Q6_K || ggml_type == SKN_TYPE_Q3_K || ggml_type == SKN_TYPE_TQ1_0 || ggml_type == SKN_TYPE_TQ2_0) ? 1
                               : (ggml_type == SKN_TYPE_Q8_0 || ggml_type == SKN_TYPE_Q2_K || ggml_type == SKN_TYPE_Q8_K) ? 3
                               : ggml_type == SKN_TYPE_IQ4_XS ? 7 : 15;
        for (int i = 0; i < 3; i++)
            SKN_REQUIRE(ctx, seg.rows[i] == 0 || (seg.w[i] && ((uintptr_t)seg.w[i] & mask) == 0), SKN_ERR_ARG,
                        "fused matvec: weights of type %d must be %d-byte aligned", ggml_type, (int)mask + 1);
    }
    SKN_REQUIRE(ctx, k > 0 && k % 256 == 0 && k <= 16384, SKN_ERR_SHAPE, "fused Q4_K matvec: unsupported k %d", k);
    skn_rope_epilogue rope;
    if (epi == SKN_EPI_ADD && rope_in && rope_in->merge_splits > 1) {
        SKN_REQUIRE(ctx, rope_in->merge_splits == 2 || rope_in->merge_splits == 4 || rope_in->merge_splits == 8, SKN_ERR_ARG,
                    "fused matvec: %d split partials (2, 4 or 8 are merged)", rope_in->merge_splits);
        SKN_REQUIRE(ctx, !norm_w && rope_in->merge_ml && rope_in->merge_head_f4 > 0 && rope_in->merge_pairs * rope_in->merge_head_f4 * 4 == k &&
                             ((uintptr_t)x & 15) == 0,
                    SKN_ERR_ARG, "fused matvec: the split partials do not cover k = %d", k);
        rope.merge_ml = rope_in->merge_ml;
        rope.merge_splits = rope_in->merge_splits;
        rope.merge_pairs = rope_in->merge_pairs;
        rope.merge_head_f4 = rope_in->merge_head_f4;
    }
    if (epi == SKN_EPI_ROPE) {
        SKN_REQUIRE(ctx, rope_in && rope_in->pos_dev && rope_in->page_table && rope_in->k_pool && rope_in->v_pool,
                    SKN_ERR_ARG, "fused Q4_K matvec: the rotary epilogue needs its cache arguments");
        rope = *rope_in;
        // (a launch may carry a subset of q, k, v: an absent matrix has no rows)
        SKN_REQUIRE(ctx, rope.head_dim > 0 && rope.head_dim % 2 == 0 && seg.rows[0] % rope.head_dim == 0 &&
                             (seg.rows[1] == 0 || seg.rows[1] == rope.n_head * rope.head_dim) &&
                             (seg.rows[2] == 0 || seg.rows[2] == rope.n_head * rope.head_dim),
                    SKN_ERR_SHAPE, "fused Q4_K matvec: q/k/v rows do not match %d heads of %d", rope.n_head,
                    rope.head_dim);
    }
    const int nb = k / 256;
#define SKN_FUSED(F)                                                                                      \
    switch ((nb + 15) / 16) {                                                                             \
        case 1: return dispatch_q4k_fused<1, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, epi, rope);       \
        case 2: return dispatch_q4k_fused<2, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, epi, rope);       \
        case 3: return dispatch_q4k_fused<3, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, epi, rope);       \
        default: return dispatch_q4k_fused<4, F>(ctx, seg, n_out, nb, x, norm_w, eps, y, epi, rope);      \
    }
    switch (ggml_type) {
        case SKN_TYPE_Q5_K: SKN_FUSED(kFmtQ5K)
        case SKN_TYPE_Q4_0: SKN_FUSED(kFmtQ40)
        case SKN_TYPE_Q4_1: SKN_FUSED(kFmtQ41)
        case SKN_TYPE_Q5_0: SKN_FUSED(kFmtQ50)
        case SKN_TYPE_Q5_1: SKN_FUSED(kFmtQ51)
        case SKN_TYPE_Q6_K: SKN_FUSED(kFmtQ6K)
        case SKN_TYPE_Q8_0: SKN_FUSED(kFmtQ80)
        case SKN_TYPE_IQ4_NL: SKN_FUSED(kFmtIQ4NL)
        case SKN_TYPE_IQ4_XS: SKN_FUSED(kFmtIQ4XS)
        case SKN_TYPE_Q2_K: SKN_FUSED(kFmtQ2K)
        case SKN_TYPE_Q3_K: SKN_FUSED(kFmtQ3K)
        case SKN_TYPE_Q8_K: SKN_FUSED(kFmtQ8K)
        case SKN_TYPE_TQ2_0: SKN_FUSED(kFmtTQ2)
        case SKN_TYPE_TQ1_0: SKN_FUSED(kFmtTQ1)
        default: SKN_FUSED(kFmtQ4K)
    }
#undef SKN_FUSED
}

// Test hook: one launch of the decoder's fused matvec, so that each fused form can be held against the oracle as an
// operation of its own.  epi 3 (rotary + cache store) appends the token at the end of sequence 0 of a one-sequence
// cache: q goes to y (fp32, rotated), k (rotated) and v into the cache as fp16.
extern "C" int skn_test_fused_matvec(skn_ctx* ctx, int ggml_type, int epi, const void* w0, int rows0, const void* w1, int rows1,
                                     const void* w2, int rows2, int k, const float* x_dev, const float* norm_w_dev, float eps,
                                     float* y_dev, skn_kv* kv, int32_t* pos_dev, float rope_base) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_test_fused_matvec: ctx is null");
    SKN_REQUIRE(ctx, epi >= SKN_EPI_STORE && epi <= SKN_EPI_ROPE && x_dev && y_dev && w0, SKN_ERR_ARG,
                "skn_test_fused_matvec: bad arguments");
    SKN_REQUIRE(ctx, ((uintptr_t)x_dev & 15) == 0 && (!norm_w_dev || ((uintptr_t)norm_w_dev & 15) == 0), SKN_ERR_ARG,
                "skn_test_fused_matvec: x and the norm weights must be 16-byte aligned");
    skn_q4k_segments seg = {{(const uint8_t*)w0, (const uint8_t*)w1, (const uint8_t*)w2}, {rows0, rows1, rows2}};
    const int n_out = epi == SKN_EPI_SWIGLU ? rows0 : rows0 + rows1 + rows2;
    if (epi == SKN_EPI_SWIGLU) SKN_REQUIRE(ctx, w1 && rows1 == rows0 && rows2 == 0, SKN_ERR_SHAPE, "skn_test_fused_matvec: gate and up must pair up");
    if (epi != SKN_EPI_ROPE) return skn_matvec_q4k_fused(ctx, seg, n_out, k, x_dev, norm_w_dev, eps, y_dev, epi, nullptr, ggml_type);
    SKN_REQUIRE(ctx, kv && pos_dev && kv->n_seq == 1, SKN_ERR_ARG, "skn_test_fused_matvec: the rotary form needs a one-sequence cache");
    const int pos = kv->len[0];
    int rc = skn_kv_reserve(ctx, kv, 0, pos + 1);
    if (rc != SKN_OK) return rc;
    SKN_HIP(ctx, hipMemcpyAsync(pos_dev, &kv->len[0], sizeof(int32_t), hipMemcpyHostToDevice, ctx->stream));
    SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));  // (the host mirror changes below)
    skn_rope_epilogue rope;
    rope.pos_dev = pos_dev;
    rope.page_table = kv->page_table_dev;
    rope.k_pool = kv->k_pool;
    rope.v_pool = kv->v_pool;
    rope.n_head = kv->n_head;
    rope.head_dim = kv->head_dim;
    rope.page_tokens = kv->page_tokens;
    rope.log2_base = log2((double)rope_base);
    // option test.rope_table: the pair frequencies come from a device table of doubles, formed on the host as the
    // decoder forms its own (the branch every decoder launch takes); otherwise the kernel forms them with exp2
    double* table = nullptr;
    if (ctx->opt_test_rope_table) {
        std::vector<double> f(kv->head_dim / 2);
        for (int i = 0; i < kv->head_dim / 2; i++) f[i] = pow((double)rope_base, -2.0 * i / kv->head_dim);
        SKN_HIP(ctx, hipMalloc((void**)&table, f.size() * sizeof(double)));
        if (hipMemcpy(table, f.data(), f.size() * sizeof(double), hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipFree(table);
            return skn_fail(ctx, SKN_ERR_HIP, "skn_test_fused_matvec: uploading the rotary frequencies failed");
        }
        rope.inv_freq = table;
    }
    rc = skn_matvec_q4k_fused(ctx, seg, n_out, k, x_dev, norm_w_dev, eps, y_dev, SKN_EPI_ROPE, &rope, ggml_type);
    if (table) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(table);
    }
    if (rc != SKN_OK) return rc;
    return skn_kv_advance_len(ctx, kv, 0, 1);
}

// Test / measurement hook: the Q4_K matvec of a three-step row (8192 < k <= 12288) with the kernel's measuring build.
extern "C" int skn_test_matvec_q4k_stamps(skn_ctx* ctx, const void* w_dev, int n, int k, const float* x_dev, float* y_dev,
                                          uint64_t* stamps_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_test_matvec_q4k_stamps: ctx is null");
    SKN_REQUIRE(ctx, w_dev && x_dev && y_dev && stamps_dev, SKN_ERR_ARG, "skn_test_matvec_q4k_stamps: null pointer");
    SKN_REQUIRE(ctx, n > 0 && k % 256 == 0 && k > 8192 && k <= 12288, SKN_ERR_SHAPE,
                "skn_test_matvec_q4k_stamps: k (%d) must be a multiple of 256 in (8192, 12288]", k);
    // (every wavefront of the last workgroup writes its eight words: the stamp buffer is 8 words per row only when
    // the rows fill whole workgroups of eight)
    SKN_REQUIRE(ctx, n % 8 == 0, SKN_ERR_SHAPE, "skn_test_matvec_q4k_stamps: n (%d) must be a multiple of 8", n);
    SKN_REQUIRE(ctx, (((uintptr_t)w_dev | (uintptr_t)x_dev) & 15) == 0 && ((uintptr_t)stamps_dev & 7) == 0, SKN_ERR_ARG,
                "skn_test_matvec_q4k_stamps: misaligned pointer");
    auto kern = matvec_q4k_kernel<3, 1, kFmtQ4K, true>;
    static bool lds_allowed[64] = {};
    int dev = 0;
    SKN_HIP(ctx, hipGetDevice(&dev));
    if (dev >= 0 && dev < 64 && !lds_allowed[dev]) {
        SKN_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        lds_allowed[dev] = true;
    }
    unsigned long long* p = reinterpret_cast<unsigned long long*>(stamps_dev);
    SKN_HIP(ctx, hipMemcpyToSymbolAsync(HIP_SYMBOL(g_matvec_stamps), &p, sizeof(p), 0, hipMemcpyHostToDevice, ctx->stream));
    const int nb = k / 256;
    const size_t lds = (size_t)3 * (16 * kXPitch * sizeof(float4) + 64 * sizeof(float2));
    skn_launch(ctx, kern, dim3((unsigned)((n + 7) / 8)), dim3(512), lds, (const uint8_t*)w_dev, x_dev, y_dev, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}

extern "C" int skn_matvec_q(skn_ctx* ctx, int ggml_type, const void* w_dev, int n, int k, const float* x_dev,
                            float* y_dev) {
    SKN_REQUIRE(nullptr, ctx != nullptr, SKN_ERR_ARG, "skn_matvec_q: ctx is null");
    SKN_REQUIRE(ctx, skn_is_quant(ggml_type), SKN_ERR_TYPE, "skn_matvec_q: ggml type %d is not supported", ggml_type);
    SKN_REQUIRE(ctx, n >= 0 && k >= 0, SKN_ERR_ARG, "skn_matvec_q: negative shape");
    int be, bb;
    skn_type_block(ggml_type, &be, &bb);
    SKN_REQUIRE(ctx, k % be == 0, SKN_ERR_SHAPE,
                "Quantized tensor row size (%d) is not a multiple of block size (%d)", k, be);
    if (n == 0) return SKN_OK;
    SKN_REQUIRE(ctx, y_dev != nullptr, SKN_ERR_ARG, "skn_matvec_q: y is null");
    if (k == 0) return skn_memset(ctx, y_dev, 0, (size_t)n * sizeof(float));
    SKN_REQUIRE(ctx, w_dev && x_dev, SKN_ERR_ARG, "skn_matvec_q: null pointer");
    SKN_REQUIRE(ctx, ((uintptr_t)x_dev & 15) == 0, SKN_ERR_ARG, "skn_matvec_q: x must be 16-byte aligned");
    SKN_REQUIRE(ctx, ((uintptr_t)w_dev & (ggml_type == SKN_TYPE_Q4_K ? 15 : ggml_type == SKN_TYPE_F32 ? 3 : 1)) == 0,
                SKN_ERR_ARG, "skn_matvec_q: weight pointer is misaligned for its block type");
    const uint8_t* w = (const uint8_t*)w_dev;
    const int nb = k / be;
    // Q5_K on the lane map of the Q4_K kernel (16-byte aligned blocks, x within the LDS of a compute unit)
    if (ggml_type == SKN_TYPE_Q5_K && ((uintptr_t)w_dev & 15) == 0 && nb <= 144 && ctx->opt_matvec_stage == 1)
        return nb > 32 ? dispatch_q4k<1, kFmtQ5K>(ctx, w, n, nb, x_dev, y_dev, 8) : dispatch_q4k<2, kFmtQ5K>(ctx, w, n, nb, x_dev, y_dev, 8);
    // Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL likewise, eight blocks standing for a superblock (rows of whole groups of eight are
    // 16-byte aligned)
    if ((ggml_type == SKN_TYPE_Q4_0 || ggml_type == SKN_TYPE_Q4_1 || ggml_type == SKN_TYPE_Q5_0 || ggml_type == SKN_TYPE_Q5_1 ||
         ggml_type == SKN_TYPE_IQ4_NL) &&
        k % 256 == 0 && ((uintptr_t)w_dev & 15) == 0 && k <= 144 * 256 && ctx->opt_matvec_stage == 1) {
        const int ng = k / 256;
#define SKN_SMALL(F) (ng > 32 ? dispatch_q4k<1, F>(ctx, w, n, ng, x_dev, y_dev, 8) : dispatch_q4k<2, F>(ctx, w, n, ng, x_dev, y_dev, 8))
        switch (ggml_type) {
            case SKN_TYPE_Q4_0: return SKN_SMALL(kFmtQ40);
            case SKN_TYPE_Q4_1: return SKN_SMALL(kFmtQ41);
            case SKN_TYPE_Q5_0: return SKN_SMALL(kFmtQ50);
            case SKN_TYPE_IQ4_NL: return SKN_SMALL(kFmtIQ4NL);
            default: return SKN_SMALL(kFmtQ51);
        }
#undef SKN_SMALL
    }
    // IQ4_XS: the superblock form of IQ4_NL on the same kernel (its blocks are 8-byte aligned)
    if (ggml_type == SKN_TYPE_IQ4_XS && ((uintptr_t)w_dev & 7) == 0 && nb <= 144 && ctx->opt_matvec_stage == 1)
        return nb > 32 ? dispatch_q4k<1, kFmtIQ4XS>(ctx, w, n, nb, x_dev, y_dev, 8) : dispatch_q4k<2, kFmtIQ4XS>(ctx, w, n, nb, x_dev, y_dev, 8);
    // Q2_K / Q3_K on the lane map of the Q6_K kernel (rows of at most four steps)
    if (ggml_type == SKN_TYPE_Q2_K && ((uintptr_t)w_dev & 3) == 0 && nb <= 64 && ctx->opt_matvec_stage == 1)
        return dispatch_runs<kRunsQ2K>(ctx, w, n, nb, x_dev, y_dev);
    if (ggml_type == SKN_TYPE_Q3_K && nb <= 64 && ctx->opt_matvec_stage == 1)
        return dispatch_runs<kRunsQ3K>(ctx, w, n, nb, x_dev, y_dev);
    if (ggml_type == SKN_TYPE_TQ2_0 && nb <= 64 && ctx->opt_matvec_stage == 1)
        return dispatch_runs<kRunsTQ2>(ctx, w, n, nb, x_dev, y_dev);
    // TQ1_0: its own lane map (blocks are 2-byte aligned)
    if (ggml_type == SKN_TYPE_TQ1_0 && ((uintptr_t)w_dev & 1) == 0 && nb <= 64 && ctx->opt_matvec_stage == 1) {
        switch ((nb + 15) / 16) {
            case 1: return launch_tq1<1>(ctx, w, n, nb, x_dev, y_dev);
            case 2: return launch_tq1<2>(ctx, w, n, nb, x_dev, y_dev);
            case 3: return launch_tq1<3>(ctx, w, n, nb, x_dev, y_dev);
            default: return launch_tq1<4>(ctx, w, n, nb, x_dev, y_dev);
        }
    }
    // Q8_K: the Q8_0 arithmetic on the Q4_K lane map (blocks are 4-byte aligned)
    if (ggml_type == SKN_TYPE_Q8_K && ((uintptr_t)w_dev & 3) == 0 && nb <= 64 && ctx->opt_matvec_stage == 1) {
        switch ((nb + 15) / 16) {
            case 1: return launch_q8k<1>(ctx, w, n, nb, x_dev, y_dev);
            case 2: return launch_q8k<2>(ctx, w, n, nb, x_dev, y_dev);
            case 3: return launch_q8k<3>(ctx, w, n, nb, x_dev, y_dev);
            default: return launch_q8k<4>(ctx, w, n, nb, x_dev, y_dev);
        }
    }
    if (!skn_is_core_quant(ggml_type)) return skn_matvec_other(ctx, ggml_type, w, n, k, x_dev, y_dev);
    if (ggml_type == SKN_TYPE_Q4_K && ctx->opt_q4k_split > 0 && nb <= 64) {
        // k split across workgroups (a measured alternative, not the default): 1 = partials merged behind a ticket,
        // 2 = floating-point atomic adds into a zeroed y
        const int slices = (nb + 15) / 16, rows = ctx->opt_q4k_rows >= 2 ? 2 : 1;
        const int groups = (n + 8 * rows - 1) / (8 * rows);
        const size_t need = (size_t)slices * n * sizeof(float) + (size_t)groups * sizeof(int);
        if (need > ctx->split_scratch_bytes) {
            SKN_HIP(ctx, hipStreamSynchronize(ctx->stream));
            if (ctx->split_scratch) SKN_HIP(ctx, hipFree(ctx->split_scratch));
            ctx->split_scratch = nullptr, ctx->split_scratch_bytes = 0;
            SKN_HIP(ctx, hipMalloc(&ctx->split_scratch, need));
            ctx->split_scratch_bytes = need;
            SKN_HIP(ctx, hipMemsetAsync(ctx->split_scratch, 0, need, ctx->stream));  // (tickets start at zero and return to it)
        }
        float* part = (float*)ctx->split_scratch;
        int* tickets = (int*)((uint8_t*)ctx->split_scratch + (size_t)slices * n * sizeof(float));
        // (the scratch is laid out for this n: another n re-zeroes the tickets' new place)
        if (ctx->split_scratch_n != n || ctx->split_scratch_slices != slices) {
            SKN_HIP(ctx, hipMemsetAsync(ctx->split_scratch, 0, ctx->split_scratch_bytes, ctx->stream));
            ctx->split_scratch_n = n, ctx->split_scratch_slices = slices;
        }
        dim3 grid((unsigned)(groups * slices)), block(512);
        if (ctx->opt_q4k_split >= 2) {
            if (slices > 1) SKN_HIP(ctx, hipMemsetAsync(y_dev, 0, (size_t)n * sizeof(float), ctx->stream));
            if (rows == 2) skn_launch(ctx, matvec_q4k_split_kernel<2, 2>, grid, block, 0, w, x_dev, y_dev, n, nb, slices, part, tickets);
            else skn_launch(ctx, matvec_q4k_split_kernel<1, 2>, grid, block, 0, w, x_dev, y_dev, n, nb, slices, part, tickets);
        } else {
            if (rows == 2) skn_launch(ctx, matvec_q4k_split_kernel<2, 1>, grid, block, 0, w, x_dev, y_dev, n, nb, slices, part, tickets);
            else skn_launch(ctx, matvec_q4k_split_kernel<1, 1>, grid, block, 0, w, x_dev, y_dev, n, nb, slices, part, tickets);
        }
        SKN_LAUNCH_CHECK(ctx);
        return SKN_OK;
    }
    if (ggml_type == SKN_TYPE_Q4_K) {
        int waves = ctx->opt_q4k_waves, rows = ctx->opt_q4k_rows;
        if (waves <= 0) waves = 8;
        if (rows <= 0) rows = nb > 32 ? 1 : 2;  // measured: long rows (three or more steps) are 2.5 % faster one per wavefront
        if (waves > 8) waves = 8;
        if (rows >= 4 && nb > 32) rows = 2;  // four rows of three or more unrolled steps do not fit the registers
        return rows >= 4   ? dispatch_q4k<4>(ctx, w, n, nb, x_dev, y_dev, waves)
               : rows >= 2 ? dispatch_q4k<2>(ctx, w, n, nb, x_dev, y_dev, waves)
                           : dispatch_q4k<1>(ctx, w, n, nb, x_dev, y_dev, waves);
    }
    if (ggml_type == SKN_TYPE_Q8_0 && nb % 2 == 0 && nb <= 512 && ((uintptr_t)w_dev & 3) == 0) {
        const int npairs = nb / 2;
        switch ((npairs + 63) / 64) {
            case 1: return launch_q80_pairs<1>(ctx, w, n, npairs, x_dev, y_dev);
            case 2: return launch_q80_pairs<2>(ctx, w, n, npairs, x_dev, y_dev);
            case 3: return launch_q80_pairs<3>(ctx, w, n, npairs, x_dev, y_dev);
            default: return launch_q80_pairs<4>(ctx, w, n, npairs, x_dev, y_dev);
        }
    }
    if (ggml_type == SKN_TYPE_Q6_K && nb <= 64) {
        switch ((nb + 15) / 16) {
            case 1: return launch_q6k<1>(ctx, w, n, nb, x_dev, y_dev);
            case 2: return launch_q6k<2>(ctx, w, n, nb, x_dev, y_dev);
            case 3: return launch_q6k<3>(ctx, w, n, nb, x_dev, y_dev);
            default: return launch_q6k<4>(ctx, w, n, nb, x_dev, y_dev);
        }
    }
    dim3 grid((unsigned)((n + 3) / 4)), block(256);
    if (ggml_type == SKN_TYPE_Q8_0)
        skn_launch(ctx, matvec_q8_0_kernel, grid, block, 0, w, x_dev, y_dev, n, nb);
    else
        skn_launch(ctx, matvec_q6_k_kernel, grid, block, 0, w, x_dev, y_dev, n, nb);
    SKN_LAUNCH_CHECK(ctx);
    return SKN_OK;
}
