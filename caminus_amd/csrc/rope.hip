// Per-head QK RMSNorm + rotary for gfx950, with the fp16 / Q8 KV row writers fused in. Replaces q3p_qk_rope and
// q3p_qk_rope_q8 (kernels/q3m_prefill.hip:534-591, the OP_OWN_ATTS prologue kernels/k3_own_atts.h:183-274) and pf_qk_nr /
// OP_QK_NR (kernels/prefill_attn.hip:106-129, kernels/k3_gguf_ops.h:1495-1518).
//
// One workgroup per token: the first wave computes the token's cos / sin row once into LDS (the reference recomputes it
// per head), then each half-wave takes one 128-wide head: lane l holds dims 4l .. 4l + 3, the NeoX partner dim i ^ 64
// sits in lane l ^ 16. Norm sum: x * x per dim, the 32-lane butterfly per 32 dims, the four group sums in order.
//
// The frequency of pair j is powf(theta_scale, j) in the reference; here it is (float)pow((double)theta_scale, j), the
// correctly rounded single-precision power, so a CPU libm that rounds powf correctly gives the same angle bits.
#include <type_traits>
#include "common.cuh"
// the fp16 rows of a prefill chunk leave as non-temporal stores (measured with every launch on cold lines: 2 % faster than plain stores)
#define RSTORE(p, v) __builtin_nontemporal_store((v), (p))

// theta_scale ** j rounded once to fp32: the product of theta_scale ** (2 ** b) over the bits of j in double-double arithmetic
// (relative error below 2 ** -95), collapsed to a double by rounding to odd, so the final conversion rounds as the exact value
// would. About 90 fp64 operations for j < 64 where the library pow() takes several hundred, on the critical path of every
// decode-sized rotary launch.
struct dd2 { double hi, lo; };
CAMX_DEV dd2 dd_mul(dd2 a, dd2 b) {
    const double p = a.hi * b.hi, e = __builtin_fma(a.hi, b.hi, -p);
    const double lo = e + (a.hi * b.lo + a.lo * b.hi), hi = p + lo;
    return {hi, lo - (hi - p)};
}
CAMX_DEV float rope_freq(float theta_scale, int j) {
    dd2 r = {1.0, 0.0}, b = {(double)theta_scale, 0.0};
    for (int n = j; n > 0; n >>= 1) {
        if (n & 1) r = dd_mul(r, b);
        if (n > 1) b = dd_mul(b, b);
    }
    if (!(__builtin_fabs(r.hi) > 1e-290 && __builtin_fabs(r.hi) < 1e290) || j < 0) return (float)pow((double)theta_scale, (double)j);
    uint64_t bits = __builtin_bit_cast(uint64_t, r.hi);
    if (r.lo != 0.0) { if ((r.lo < 0.0) != (r.hi < 0.0)) bits -= 1; bits |= 1; }
    return (float)__builtin_bit_cast(double, bits);
}

struct RopeArgs {
    const void * qkv; int ldq, nh, nkv;       // fp32, or bf16 (BF16IN) widened exactly
    const float * par;               // q_norm[128] | k_norm[128] | theta_scale | eps | (yarn: freq[64] | mscale)
    int pos0; const int32_t * pos;   // token t is at pos ? pos[t] : pos0 + t
    uint16_t * q16;                  // fp16 [n][nh][128]
    void * cache;                    // fp16 rows [K (nkv*128) | V] or Q8 rows
    int * err;
    const int32_t * page_table; int pt_stride, page, n_pages;   // paged addressing (null: row = position)
    int n;
    int rows;                        // unpaged: rows of the cache when positions come from the caller's array (0: not checked here)
    const int32_t * posb;            // the tape's device-resident position: token t is at posb[0] + t (pos and pos0 unused)
};
CAMX_DEV int rope_pos(const RopeArgs & a, int t) { return a.pos ? a.pos[t] : (a.posb ? a.posb[0] : a.pos0) + t; }

// TPW tokens per workgroup: 1 for decode-sized batches (wave 0 computes the token's cos / sin row); 4 for prefill chunks, where
// wave w computes token w's row, one barrier publishes all four, and each wave then walks the tokens with the next token's
// (or next pass's) loads in flight during the current one's arithmetic.
template <int S> CAMX_DEV float half_lane_bcast(float v) {   // every lane of a 32-lane half reads the half's lane S
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x00 | (S << 5)));
}

// NW waves per workgroup and QR_STEPS wave steps per pass: 4 x 5 (a pass of 40 heads, ten per wave), or 10 x 2 for batches too small to
// fill the chip, where a token's heads spread over more waves and each wave's chain of steps is two long instead of five.
template <bool YARN, bool Q8, bool BF16IN, int TPW, int NW = 4, int QR_STEPS = 5>
__global__ void __launch_bounds__(NW * 64) qk_rope_tokens(RopeArgs a) {
    __shared__ __attribute__((aligned(16))) float rc[TPW][64];
    __shared__ __attribute__((aligned(16))) float rs[TPW][64];
    const int t0 = blockIdx.x * TPW, tid = threadIdx.x, lraw = tid & 63, lane = slot_of(lraw), l = lane & 31, wave = tid >> 6;
    // items: heads 0 .. nh + nkv - 1 take norm + rotary, items nh + nkv .. nh + 2 nkv - 1 are the V heads. A wave step is two
    // heads (one per half-wave); the loads of up to QR_STEPS steps (one pass) are issued together, and before the cos / sin
    // rows are computed, so a decode token pays one memory round trip, not one per head.
    const int items = a.nh + 2 * a.nkv;
    constexpr int HS = 2 * NW;                                          // heads per wave step of the workgroup
    const int npass = (items + HS * QR_STEPS - 1) / (HS * QR_STEPS);
    const int it_w = wave * 2 + (lane >> 5);                            // this half-wave's head inside a step of HS heads
    f32x4 xin[QR_STEPS], xnext[QR_STEPS];
    auto load = [&](f32x4 (&buf)[QR_STEPS], int tok, int base) {
        const int tk = tok < a.n ? tok : 0;
        const float * row = (const float *)a.qkv + (size_t)tk * a.ldq;
        const uint16_t * rowb = (const uint16_t *)a.qkv + (size_t)tk * a.ldq;
#pragma unroll
        for (int s = 0; s < QR_STEPS; s++) {
            const int it = base + HS * s + it_w;
            const int hy = it < items ? it : 0;
            buf[s] = BF16IN ? unpack_bf16x4(*(const u32x2 *)(rowb + (size_t)hy * 128 + 4 * l)) : *(const f32x4 *)(row + (size_t)hy * 128 + 4 * l);
        }
    };
    load(xin, t0, 0);
    const f32x4 wq = *(const f32x4 *)(a.par + 4 * l), wk = *(const f32x4 *)(a.par + 128 + 4 * l);
    const float eps = a.par[257];
    for (int tr = wave; tr < TPW; tr += NW) {                               // the tokens whose cos / sin rows this wave computes
        if (t0 + tr < a.n) {
            const int pos = rope_pos(a, t0 + tr);
            float c, s;
            if (YARN) { const float theta = (float)pos * a.par[258 + lraw], ms = a.par[322]; c = cosf(theta) * ms; s = sinf(theta) * ms; }
            else { const float theta = (float)pos * rope_freq(a.par[256], lraw); c = cosf(theta); s = sinf(theta); }
            rc[tr][lraw] = c; rs[tr][lraw] = s;
        }
    }
    __syncthreads();
    const size_t M = (size_t)a.nkv * 128;
    const size_t rb = Q8 ? 2 * (M / 32) * 34 : 4 * M;
    const bool lo = l < 16;
    for (int it_tp = 0; it_tp < TPW * npass; it_tp++) {
        const int ti = it_tp / npass, base = (it_tp - ti * npass) * HS * QR_STEPS, t = t0 + ti;
        if (t >= a.n) break;
        if (it_tp + 1 < TPW * npass) { const int tn = (it_tp + 1) / npass; load(xnext, t0 + tn, ((it_tp + 1) - tn * npass) * HS * QR_STEPS); }
        const int pos = rope_pos(a, t);
        uint8_t * cw = nullptr;
        // a position outside the sequence's table row (paged) or outside the cache (unpaged): bit 1, that sequence's row is not written
        const bool span = pos >= 0 && (a.page_table ? pos / a.page < a.pt_stride : (a.rows == 0 || pos < a.rows));
        if (!span) { if (a.err && tid == 0 && base == 0) atomicOr(a.err, 1); }
        else if (a.page_table) {
            const int pg = a.page_table[(size_t)t * a.pt_stride + pos / a.page];
            if (pg < 0 || pg >= a.n_pages) { if (tid == 0 && base == 0) atomicOr(a.err, 8); }
            else cw = (uint8_t *)a.cache + ((size_t)pg * a.page + (size_t)(pos % a.page)) * rb;
        } else cw = (uint8_t *)a.cache + (size_t)pos * rb;
        const f32x4 c4 = *(const f32x4 *)(rc[ti] + 4 * (l & 15)), s4 = *(const f32x4 *)(rs[ti] + 4 * (l & 15));
        // the sums of squares of all steps first (every lane active), then ONE IEEE sqrt + divide per half-wave for all of
        // them: lane s of a half-wave takes step s, and the half-wave reads it back
        float tot[QR_STEPS];
#pragma unroll
        for (int st = 0; st < QR_STEPS; st++) {
            const f32x4 x = xin[st];
            f32x4 sq; sq.x = x.x * x.x; sq.y = x.y * x.y; sq.z = x.z * x.z; sq.w = x.w * x.w;
            tot[st] = half_groups_in_order<4>(group32_sum(sq), lane & 32);
        }
        float tv = tot[0];
#pragma unroll
        for (int st = 1; st < QR_STEPS; st++) tv = (lraw & 31) == st ? tot[st] : tv;
        const float sc = rsqrt_exact(tv / 128 + eps);
        float scl[QR_STEPS];
        static_assert(QR_STEPS <= 5, "the broadcasts below are written out for at most five steps");
        scl[0] = half_lane_bcast<0>(sc);
        if (QR_STEPS > 1) scl[1 % QR_STEPS] = half_lane_bcast<1>(sc);
        if (QR_STEPS > 2) scl[2 % QR_STEPS] = half_lane_bcast<2>(sc);
        if (QR_STEPS > 3) scl[3 % QR_STEPS] = half_lane_bcast<3>(sc);
        if (QR_STEPS > 4) scl[4 % QR_STEPS] = half_lane_bcast<4>(sc);
#pragma unroll
        for (int st = 0; st < QR_STEPS; st++) {
            if (base + HS * st + wave * 2 >= items) break;               // wave-uniform: neither half-wave has a head
            const int it = base + HS * st + it_w;
            const bool active = it < items;
            const int hy = active ? it : 0;
            const f32x4 x = xin[st];
            if (hy >= a.nh + a.nkv) {                       // a V head: fp16 copy, or fp16-rounded then Q8 blocks
                const int g = hy - a.nh - a.nkv;
                if (Q8) {
                    f32x4 v; v.x = f16r(x.x); v.y = f16r(x.y); v.z = f16r(x.z); v.w = f16r(x.w);
                    kv_q8_emit(v, cw + (M / 32 + (size_t)g * 4 + (l >> 3)) * 34, l & 7, a.err, active && cw != nullptr);
                } else if (active && cw) *(u32x2 *)((uint16_t *)cw + M + (size_t)g * 128 + 4 * l) = pack_f16x4(x);
                continue;
            }
            const bool isq = hy < a.nh;
            const f32x4 wn = isq ? wq : wk;
            const float scale = scl[st];
            f32x4 y1; y1.x = (scale * x.x) * wn.x; y1.y = (scale * x.y) * wn.y; y1.z = (scale * x.z) * wn.z; y1.w = (scale * x.w) * wn.w;
            f32x4 p; p.x = lane_xor16(y1.x); p.y = lane_xor16(y1.y); p.z = lane_xor16(y1.z); p.w = lane_xor16(y1.w);
            // dims below 64: fma(x0, c, -(x1 s)); dims from 64: fma(x1, c, x0 s), with x0 the low and x1 the high dim of the pair
            f32x4 y;
            y.x = __builtin_fmaf(y1.x, c4.x, lo ? -(p.x * s4.x) : p.x * s4.x); y.y = __builtin_fmaf(y1.y, c4.y, lo ? -(p.y * s4.y) : p.y * s4.y);
            y.z = __builtin_fmaf(y1.z, c4.z, lo ? -(p.z * s4.z) : p.z * s4.z); y.w = __builtin_fmaf(y1.w, c4.w, lo ? -(p.w * s4.w) : p.w * s4.w);
            if (Q8) {
                y.x = f16r(y.x); y.y = f16r(y.y); y.z = f16r(y.z); y.w = f16r(y.w);
                y = hadamard128_l4(y, l, true);
            }
            if (isq) {
                if (Q8) { asm volatile("" : "+v"(y.x), "+v"(y.y), "+v"(y.z), "+v"(y.w)); }   // fp32 product first, then fp16
                if (active) *(u32x2 *)(a.q16 + ((size_t)t * a.nh + hy) * 128 + 4 * l) = pack_f16x4(y);
            } else {
                const int g = hy - a.nh;
                if (Q8) kv_q8_emit(y, cw + ((size_t)g * 4 + (l >> 3)) * 34, l & 7, a.err, active && cw != nullptr);
                else if (active && cw) *(u32x2 *)((uint16_t *)cw + (size_t)g * 128 + 4 * l) = pack_f16x4(y);
            }
        }
#pragma unroll
        for (int st = 0; st < QR_STEPS; st++) xin[st] = xnext[st];
    }
}

// ---- the bf16 prefill form: 8 dims per lane, 16 lanes per head, 4 heads per wave instruction -----------------------------------
// A token's q | k | v heads are contiguous 256-byte runs of bf16, so one 128-bit load per lane covers four heads (1 KiB per
// wave instruction) and the fp16 results leave as 128-bit stores. Lane l (of 16) holds dims 8 l .. 8 l + 7: the 32-thread
// butterfly of the norm sum is lane ^ 2, lane ^ 1 (quad permutes) and three in-register levels (the same pairs in the same
// order as thread xor 16, 8, 4, 2, 1), the four group sums are fetched with bit-mask swizzles and added in order, and the
// NeoX partner dim i ^ 64 sits in lane l ^ 8 (row_ror:8). Each wave issues the loads of all its heads (up to STEPS
// wave steps) before the token's cos / sin row is computed, so the row's bytes are in flight during the trigonometry.
CAMX_DEV float swz_group(float v, int j) {        // every lane of a 16-lane row reads the row's lane 4 j + (lane & 3)
    const int i = __builtin_bit_cast(int, v);
    switch (j) {
    case 0: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(i, 0x13 | (0 << 5)));
    case 1: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(i, 0x13 | (4 << 5)));
    case 2: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(i, 0x13 | (8 << 5)));
    default: return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(i, 0x13 | (12 << 5)));
    }
}
CAMX_DEV float dpp_xor1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)); }
CAMX_DEV float dpp_xor2(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)); }
CAMX_DEV float dpp_ror8(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false)); }
CAMX_DEV uint32_t pack_f16x2(float lo, float hi) {
    asm volatile("" : "+v"(lo), "+v"(hi));                       // already rounded to fp32: never fused with the producer
    const f32x2 in = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, f16x2));
}

// v + (v of lane ^ 1), v + (v of lane ^ 2), (v of lane ^ 8 inside its row of 16) * m: the cross-lane move rides on the
// arithmetic instruction as a DPP source modifier (every lane is active wherever these are used)
template <int CTRL> CAMX_DEV float dpp_full(float v) {   // full row / bank masks and bound_ctrl: the backend folds the move into its user
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
CAMX_DEV float add_xor1(float v) { return dpp_full<0xB1>(v) + v; }
CAMX_DEV float add_xor2(float v) { return dpp_full<0x4E>(v) + v; }
CAMX_DEV float mul_ror8(float v, float m) { return dpp_full<0x128>(v) * m; }
template <int S> CAMX_DEV float row_lane_bcast(float v) {   // every lane of a 16-lane row reads the row's lane S
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x10 | (S << 5)));
}

// the orthonormal 128-point Walsh-Hadamard transform of a head held by 16 lanes x 8 registers (element 8 l + k): stages
// h = 1, 2, 4 pair registers, h = 8 .. 64 pair lanes l ^ 1 .. l ^ 8, in that order (the order of hadamard128_l4: same sums,
// same bits); the upper lane of a pair flips its sign and both add the partner's value; then times 0x1.6a09e6p-4f
CAMX_DEV void hadamard128_w8(float (&e)[8], int l16) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
        for (int k = 0; k < 8; k++)
            if (!(k & h)) { const float a = e[k], b = e[k + h]; e[k] = a + b; e[k + h] = a - b; }
#define W8_STAGE(BIT, PARTNER)                                                                                   \
    {                                                                                                              \
        const uint32_t m = (l16 & BIT) ? 0x80000000u : 0u;                                                         \
        _Pragma("unroll") for (int k = 0; k < 8; k++) {                                                            \
            const float own = e[k];                                                                                \
            e[k] = PARTNER(own) + __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, own) ^ m);                \
        }                                                                                                          \
    }
#define W8_XOR4(x) __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x101F))
    W8_STAGE(1, dpp_full<0xB1>) W8_STAGE(2, dpp_full<0x4E>) W8_STAGE(4, W8_XOR4) W8_STAGE(8, dpp_full<0x128>)
#undef W8_XOR4
#undef W8_STAGE
#pragma unroll
    for (int k = 0; k < 8; k++) e[k] *= 0x1.6a09e6p-4f;
}
// kv_q8_emit for a block of 32 values held by 4 lanes x 8 registers (sub = lane & 3): the same decisions and bytes
CAMX_DEV void kv_q8_emit_w8(const float (&v)[8], uint8_t * blk, int sub, int * err, bool active) {
    bool fin = true;
    float m = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) { fin = fin && __builtin_isfinite(v[k]); m = fmaxf(m, fabsf(v[k])); }
    m = fin ? m : INFINITY;
    m = fmaxf(m, dpp_xor1(m)); const float amax = fmaxf(m, dpp_xor2(m));
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const _Float16 stored = (_Float16)d;
    const bool refuse = !__builtin_isfinite(amax) ||
                        (amax != 0.0f && (d == 0.0f || !__builtin_isfinite(d) || !__builtin_isfinite(inv) || !__builtin_isfinite((float)stored)));
    if (!active) return;
    if (refuse) { if (sub == 0) atomicOr(err, 2); return; }
    const f32x4 t0 = {v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv}, t1 = {v[4] * inv, v[5] * inv, v[6] * inv, v[7] * inv};
    const uint32_t q0 = pack_round_i8x4(t0), q1 = pack_round_i8x4(t1);
    uint16_t * o = (uint16_t *)(blk + 2 + 8 * sub);
    o[0] = (uint16_t)q0; o[1] = (uint16_t)(q0 >> 16); o[2] = (uint16_t)q1; o[3] = (uint16_t)(q1 >> 16);
    if (sub == 0) *(uint16_t *)blk = __builtin_bit_cast(uint16_t, stored);
}

// TPW tokens per workgroup. With four, wave w computes the cos / sin row of token w while every wave's first loads are in
// flight, one barrier publishes the four rows, and then each wave walks the four tokens on its own, loading token i + 1's
// heads before it does token i's arithmetic. With one (small batches), wave 0 computes the row.
// F32IN: fp32 rows (two 128-bit loads per lane and step), else bf16 rows (one). STEPS wave steps of 16 heads per pass.
// Q8: the Q8 cache rows (K through the Hadamard transform, V unrotated, both from fp16-rounded values) and q16 = fp16 of
// the transformed q, as in qk_rope_tokens.
template <bool YARN, int TPW, bool F32IN, int STEPS, bool Q8>
__global__ void __launch_bounds__(256) qk_rope_wide_tokens(RopeArgs a) {
    __shared__ __attribute__((aligned(16))) float rc[TPW][64];
    __shared__ __attribute__((aligned(16))) float rs[TPW][64];
    __shared__ __attribute__((aligned(16))) float nrm[256];                  // q_norm | k_norm
    const int t0 = blockIdx.x * TPW, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, hq = lane >> 4;
    const int items = a.nh + 2 * a.nkv, nqk = a.nh + a.nkv;
    const size_t M = (size_t)a.nkv * 128;
    const int lo = 128 * hq + 8 * l16;                                      // this lane's element offset inside a wave step
    const int nchunk = (items + 16 * STEPS - 1) / (16 * STEPS);       // a row longer than 80 heads takes several passes
    constexpr int NW = F32IN ? 2 : 1;
    u32x4 xin[STEPS][NW], xnext[STEPS][NW];
    auto load = [&](u32x4 (&buf)[STEPS][NW], int tok, int base) {
#pragma unroll
        for (int s = 0; s < STEPS; s++) {                                // wave step s: heads base + 16 s + 4 wave + (0 .. 3)
            const int h0 = base + 16 * s + 4 * wave;
            const bool ok = tok < a.n && h0 + hq < items;
#pragma unroll
            for (int w = 0; w < NW; w++) buf[s][w] = (u32x4){0u, 0u, 0u, 0u};
            if (ok) {
                if (F32IN) {
                    const float * p = (const float *)a.qkv + (size_t)tok * a.ldq + (size_t)h0 * 128 + lo;
                    buf[s][0] = __builtin_nontemporal_load((const u32x4 *)p); buf[s][NW - 1] = __builtin_nontemporal_load((const u32x4 *)(p + 4));
                } else buf[s][0] = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)a.qkv + (size_t)tok * a.ldq + (size_t)h0 * 128 + lo));
            }
        }
    };
    load(xin, t0, 0);
    nrm[tid] = a.par[tid];
    for (int tr = wave; tr < TPW; tr += 4) {                               // the tokens whose cos / sin rows this wave computes
        if (t0 + tr < a.n) {
            const int pos = rope_pos(a, t0 + tr);
            float c, sn;
            if (YARN) { const float theta = (float)pos * a.par[258 + lane], ms = a.par[322]; c = cosf(theta) * ms; sn = sinf(theta) * ms; }
            else { const float theta = (float)pos * rope_freq(a.par[256], lane); c = cosf(theta); sn = sinf(theta); }
            rc[tr][lane] = c; rs[tr][lane] = sn;
        }
    }
    __syncthreads();
    const float eps = a.par[257];
    for (int it = 0; it < TPW * nchunk; it++) {
        const int ti = it / nchunk, base = (it - ti * nchunk) * 16 * STEPS, t = t0 + ti;
        if (t >= a.n) break;
        if (it + 1 < TPW * nchunk) { const int tn = (it + 1) / nchunk; load(xnext, t0 + tn, ((it + 1) - tn * nchunk) * 16 * STEPS); }
        const int pos = rope_pos(a, t);
        const bool span = pos >= 0 && (a.rows == 0 || pos < a.rows);          // (wave-uniform) outside the cache: bit 1, no row written
        if (!span && a.err && tid == 0 && base == 0) atomicOr(a.err, 1);
        uint16_t * cw = (uint16_t *)a.cache + (size_t)(span ? pos : 0) * 2 * M;
        uint16_t * qw = a.q16 + (size_t)t * a.nh * 128;
        const int j0 = 8 * (l16 & 7);
        f32x4 c4[2], s4[2];
        c4[0] = *(const f32x4 *)(rc[ti] + j0); c4[1] = *(const f32x4 *)(rc[ti] + j0 + 4);
        s4[0] = *(const f32x4 *)(rs[ti] + j0); s4[1] = *(const f32x4 *)(rs[ti] + j0 + 4);
        if (l16 < 8) { s4[0] = -s4[0]; s4[1] = -s4[1]; }                    // dims below 64 take -(x1 s): the sign moves into s
        // phase 1: the sum of squares of every step's heads (V heads included: their sums are never used)
        float x[STEPS][8], tot[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            if (F32IN) {
#pragma unroll
                for (int p = 0; p < 4; p++) { const uint32_t b0 = xin[s][0][p], b1 = xin[s][NW - 1][p]; x[s][p] = __builtin_bit_cast(float, b0); x[s][4 + p] = __builtin_bit_cast(float, b1); }
            } else {
#pragma unroll
                for (int p = 0; p < 4; p++) { const uint32_t b = xin[s][0][p]; x[s][2 * p] = __builtin_bit_cast(float, b << 16); x[s][2 * p + 1] = __builtin_bit_cast(float, b & 0xffff0000u); }
            }
            float sq[8];
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = x[s][k] * x[s][k];
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor2(sq[k]);            // thread ^ 16
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor1(sq[k]);            // thread ^ 8
            const float b0 = sq[0] + sq[4], b1 = sq[1] + sq[5], b2 = sq[2] + sq[6], b3 = sq[3] + sq[7];   // thread ^ 4
            const float e0 = b0 + b2, e1 = b1 + b3;                         // thread ^ 2
            const float g = e0 + e1;                                        // thread ^ 1
            tot[s] = ((swz_group(g, 0) + swz_group(g, 1)) + swz_group(g, 2)) + swz_group(g, 3);
        }
        // phase 2: one IEEE sqrt + divide per row for all steps: lane s of a row takes step s, the row reads it back
        float tv = tot[0];
#pragma unroll
        for (int s = 1; s < STEPS; s++) tv = l16 == s ? tot[s] : tv;
        const float sc = rsqrt_exact(tv / 128 + eps);
        float scale[STEPS];
        static_assert(STEPS <= 5, "the broadcasts below are written out for at most five steps");
        scale[0] = row_lane_bcast<0>(sc);
        if (STEPS > 1) scale[1 % STEPS] = row_lane_bcast<1>(sc);
        if (STEPS > 2) scale[2 % STEPS] = row_lane_bcast<2>(sc);
        if (STEPS > 3) scale[3 % STEPS] = row_lane_bcast<3>(sc);
        if (STEPS > 4) scale[4 % STEPS] = row_lane_bcast<4>(sc);
        // phase 3: scale, rotate, convert, store
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int h0 = base + 16 * s + 4 * wave;                        // wave-uniform
            if (h0 >= items) break;
            u32x4 out;
            if constexpr (Q8) {
                const int h = h0 + hq;                                      // this row of 16 lanes: one head
                const bool isq = h < a.nh, isv = h >= nqk, active = h < items;
                uint8_t * cwb = (uint8_t *)a.cache + (size_t)(span ? pos : 0) * (2 * (M / 32) * 34);
                float v8[8];
                if (isv) {
#pragma unroll
                    for (int k = 0; k < 8; k++) v8[k] = f16r(x[s][k]);
                } else {
                    const float * wp = nrm + (isq ? 0 : 128) + 8 * l16;
                    const f32x4 w0 = *(const f32x4 *)wp, w1 = *(const f32x4 *)(wp + 4);
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const float y1 = (scale[s] * x[s][k]) * (k < 4 ? w0[k] : w1[k - 4]);
                        v8[k] = f16r(__builtin_fmaf(y1, k < 4 ? c4[0][k] : c4[1][k - 4], mul_ror8(y1, k < 4 ? s4[0][k] : s4[1][k - 4])));
                    }
                    hadamard128_w8(v8, l16);
                }
                if (isq) {
#pragma unroll
                    for (int p = 0; p < 4; p++) out[p] = pack_f16x2(v8[2 * p], v8[2 * p + 1]);
                    if (active) *(u32x4 *)(qw + (size_t)h * 128 + 8 * l16) = out;
                } else {
                    const size_t b = isv ? M / 32 + (size_t)(h - nqk) * 4 + (l16 >> 2) : (size_t)(h - a.nh) * 4 + (l16 >> 2);
                    kv_q8_emit_w8(v8, cwb + b * 34, l16 & 3, a.err, active && span);
                }
                continue;
            }
            if (h0 >= nqk) {                                                // V heads only: fp16 copy
#pragma unroll
                for (int p = 0; p < 4; p++) out[p] = pack_f16x2(x[s][2 * p], x[s][2 * p + 1]);
                if (h0 + hq < items && span) RSTORE((u32x4 *)(cw + M + (size_t)(h0 - nqk) * 128 + lo), out);
                continue;
            }
            const bool allq = h0 + 3 < a.nh, allk = h0 >= a.nh && h0 + 3 < nqk;
            const int h = h0 + hq;
            const bool isq = h < a.nh, isv = h >= nqk;
            const float * wp = nrm + ((allq || (!allk && isq)) ? 0 : 128) + 8 * l16;
            const f32x4 w0 = *(const f32x4 *)wp, w1 = *(const f32x4 *)(wp + 4);
            float y[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float y1 = (scale[s] * x[s][k]) * (k < 4 ? w0[k] : w1[k - 4]);
                y[k] = __builtin_fmaf(y1, k < 4 ? c4[0][k] : c4[1][k - 4], mul_ror8(y1, k < 4 ? s4[0][k] : s4[1][k - 4]));
            }
            if (allq) {
#pragma unroll
                for (int p = 0; p < 4; p++) out[p] = pack_f16x2(y[2 * p], y[2 * p + 1]);
                RSTORE((u32x4 *)(qw + (size_t)h0 * 128 + lo), out);
            } else if (allk) {
#pragma unroll
                for (int p = 0; p < 4; p++) out[p] = pack_f16x2(y[2 * p], y[2 * p + 1]);
                if (span) RSTORE((u32x4 *)(cw + (size_t)(h0 - a.nh) * 128 + lo), out);
            } else {                                                        // a step that straddles q | k | v or the end of the row
#pragma unroll
                for (int k = 0; k < 8; k++) if (isv) y[k] = x[s][k];
#pragma unroll
                for (int p = 0; p < 4; p++) out[p] = pack_f16x2(y[2 * p], y[2 * p + 1]);
                if (h < items && (isq || span)) {
                    uint16_t * dst = isq ? qw + (size_t)h * 128 : (isv ? cw + M + (size_t)(h - nqk) * 128 : cw + (size_t)(h - a.nh) * 128);
                    RSTORE((u32x4 *)(dst + 8 * l16), out);
                }
            }
        }
#pragma unroll
        for (int s = 0; s < STEPS; s++)
#pragma unroll
            for (int w = 0; w < NW; w++) xin[s][w] = xnext[s][w];
    }
}

// ---- the same arithmetic for the aligned shape of a dense bf16 prefill chunk, written straight-line -----------------------------
// Rows of exactly 16 STEPS heads (STEPS <= 5) with nh and nkv multiples of 4, so a wave step of four heads is wholly q, k or v and
// no lane is ever predicated; positions pos0 + t. TPW tokens per workgroup, all their loads issued before anything else (one
// burst of reads per wave, then its arithmetic, then one burst of writes), the norm weights and the tokens' cos / sin rows in LDS.
// The operations and their order are qk_rope_wide_tokens': same bits. F32IN: fp32 rows (two 128-bit loads per lane and step) of up to 48
// heads, the last step possibly short (16384 tokens x 40 heads: 92 -> 86.5 us against the pipelined kernel).
// GEN: any addressing the token kernels take (a position per token or a device-resident base, a page table, a bound on the cache's rows),
// with their refusals: a row that is refused is not written and sets its error bit; q16 is written for every token.
template <bool YARN, int STEPS, int TPW, bool F32IN = false, bool Q8 = false, bool GEN = false>
__global__ void __launch_bounds__(256) qk_rope_chunk(RopeArgs a) {
    __shared__ __attribute__((aligned(16))) float rc[TPW][64];
    __shared__ __attribute__((aligned(16))) float rs[TPW][64];
    __shared__ __attribute__((aligned(16))) float nrm[256];                  // q_norm | k_norm
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, hq = lane >> 4;
    const int t0 = blockIdx.x * TPW;
    const int nqk = a.nh + a.nkv, items = a.nh + 2 * a.nkv;             // (F32IN: the last step may hold fewer than 16 heads; a wave's four are all there or not)
    const size_t M = (size_t)a.nkv * 128;
    const int lo = 128 * hq + 8 * l16;                                      // this lane's element offset inside a wave step
    constexpr int NW = F32IN ? 2 : 1;
    u32x4 xin[TPW][STEPS][NW];
    // fp32 rows: a lane's eight values are 32 bytes, so loading them straight into its registers takes two requests that each use half of
    // every line. The wave's four heads of a step (2 KiB) go to LDS instead, 16 bytes per lane with neighbouring lanes on neighbouring
    // addresses (whole lines per request, no registers held while they fly), and each lane reads its eight values from there.
    // (not for the Q8 rows, whose time is their arithmetic: the 24 KiB per workgroup cost them resident waves, 94 -> 101 us at 16384 tokens)
    constexpr bool STAGE = F32IN && !Q8;
    __shared__ __attribute__((aligned(16))) float stg[STAGE ? TPW * STEPS * 2048 : 4];
#pragma unroll
    for (int ti = 0; ti < TPW; ti++) {
        const int tk = t0 + ti < a.n ? t0 + ti : a.n - 1;
        const size_t e = (size_t)tk * a.ldq + 512 * wave + lo;               // heads 16 s + 4 wave .. + 3
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            if (F32IN && !STAGE) {
                xin[ti][s][0] = xin[ti][s][NW - 1] = (u32x4){0u, 0u, 0u, 0u};
                if (16 * s + 4 * wave < items) {
                    const float * p = (const float *)a.qkv + e + 2048 * s;
                    xin[ti][s][0] = __builtin_nontemporal_load((const u32x4 *)p); xin[ti][s][NW - 1] = __builtin_nontemporal_load((const u32x4 *)(p + 4));
                }
            } else if (STAGE) {
                if (16 * s + 4 * wave < items) {
                    const float * p = (const float *)a.qkv + (size_t)tk * a.ldq + 2048 * s + 512 * wave + 4 * lane;
                    float * d = stg + (ti * STEPS + s) * 2048 + 512 * wave;
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p, (__attribute__((address_space(3))) void *)d, 16, 0, 2);
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p + 256), (__attribute__((address_space(3))) void *)(d + 256), 16, 0, 2);
                }
            } else xin[ti][s][0] = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)a.qkv + e + 2048 * s));
        }
    }
    // GEN: the tokens' positions and page ids are two dependent loads per token; they start here, behind the rows' loads, and not when
    // the token's turn comes
    [[maybe_unused]] int posv[TPW], pgv[TPW];
    if constexpr (GEN) {
#pragma unroll
        for (int ti = 0; ti < TPW; ti++) posv[ti] = rope_pos(a, t0 + ti < a.n ? t0 + ti : a.n - 1);
#pragma unroll
        for (int ti = 0; ti < TPW; ti++) {
            pgv[ti] = 0;
            if (a.page_table && posv[ti] >= 0 && posv[ti] / a.page < a.pt_stride)
                pgv[ti] = a.page_table[(size_t)(t0 + ti < a.n ? t0 + ti : a.n - 1) * a.pt_stride + posv[ti] / a.page];
        }
    }
    nrm[tid] = a.par[tid];
    if (wave < TPW) {                                                       // wave w: the cos / sin row of token t0 + w
        const int tw = t0 + wave < a.n ? t0 + wave : a.n - 1;
        const int pos = GEN ? rope_pos(a, tw) : a.pos0 + tw;
        float c, sn;
        if (YARN) { const float theta = (float)pos * a.par[258 + lane], ms = a.par[322]; c = cosf(theta) * ms; sn = sinf(theta) * ms; }
        else { const float theta = (float)pos * rope_freq(a.par[256], lane); c = cosf(theta); sn = sinf(theta); }
        rc[wave][lane] = c; rs[wave][lane] = sn;
    }
    if (STAGE) __builtin_amdgcn_s_waitcnt(0x0f70);                          // vmcnt(0): the wave's own heads have landed in LDS
    __syncthreads();
    if (STAGE) {
#pragma unroll
        for (int ti = 0; ti < TPW; ti++)
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                xin[ti][s][0] = xin[ti][s][NW - 1] = (u32x4){0u, 0u, 0u, 0u};
                if (16 * s + 4 * wave < items) {
                    const float * q = stg + (ti * STEPS + s) * 2048 + 512 * wave + lo;
                    xin[ti][s][0] = *(const u32x4 *)q; xin[ti][s][NW - 1] = *(const u32x4 *)(q + 4);
                }
            }
    }
    const float eps = a.par[257];
#pragma unroll
    for (int ti = 0; ti < TPW; ti++) {
        const int t = t0 + ti;
        if (t >= a.n) break;
        int pos = a.pos0 + t;
        if constexpr (GEN) pos = posv[ti];
        bool span = true;                                                   // (wave-uniform) the token's cache row may be written
        size_t rowi = (size_t)pos;
        if constexpr (GEN) {
            span = pos >= 0 && (a.page_table ? pos / a.page < a.pt_stride : (a.rows == 0 || pos < a.rows));
            if (!span) { if (a.err && tid == 0) atomicOr(a.err, 1); }
            else if (a.page_table) {
                const int pg = pgv[ti];
                if (pg < 0 || pg >= a.n_pages) { if (tid == 0) atomicOr(a.err, 8); span = false; }
                else rowi = (size_t)pg * a.page + (size_t)(pos % a.page);
            }
            if (!span) rowi = 0;
        }
        uint16_t * cw = (uint16_t *)a.cache + rowi * 2 * M;
        uint16_t * qw = a.q16 + (size_t)t * a.nh * 128;
        const int j0 = 8 * (l16 & 7);
        f32x4 c4[2], s4[2];
        c4[0] = *(const f32x4 *)(rc[ti] + j0); c4[1] = *(const f32x4 *)(rc[ti] + j0 + 4);
        s4[0] = *(const f32x4 *)(rs[ti] + j0); s4[1] = *(const f32x4 *)(rs[ti] + j0 + 4);
        if (l16 < 8) { s4[0] = -s4[0]; s4[1] = -s4[1]; }                    // dims below 64 take -(x1 s): the sign moves into s
        // phase 1: the sum of squares of every q / k step (thread ^ 16, ^ 8 across lanes, ^ 4, ^ 2, ^ 1 in registers, four groups in order)
        float tot[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            tot[s] = 1.0f;
            if (16 * s + 4 * wave >= nqk) continue;                         // (wave-uniform) V heads: no norm
            float sq[8];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (F32IN) {
                    const uint32_t b0 = xin[ti][s][0][p], b1 = xin[ti][s][NW - 1][p];
                    const float x0 = __builtin_bit_cast(float, b0), x1 = __builtin_bit_cast(float, b1);
                    sq[p] = x0 * x0; sq[4 + p] = x1 * x1;
                } else {
                    const uint32_t b = xin[ti][s][0][p];
                    const float x0 = __builtin_bit_cast(float, b << 16), x1 = __builtin_bit_cast(float, b & 0xffff0000u);
                    sq[2 * p] = x0 * x0; sq[2 * p + 1] = x1 * x1;
                }
            }
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor2(sq[k]);
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor1(sq[k]);
            const float b0 = sq[0] + sq[4], b1 = sq[1] + sq[5], b2 = sq[2] + sq[6], b3 = sq[3] + sq[7];
            const float e0 = b0 + b2, e1 = b1 + b3;
            const float g = e0 + e1;
            tot[s] = ((swz_group(g, 0) + swz_group(g, 1)) + swz_group(g, 2)) + swz_group(g, 3);
        }
        // phase 2: one IEEE sqrt + divide per row for all steps: lane s of a row takes step s, the row reads it back
        float tv = tot[0];
#pragma unroll
        for (int s = 1; s < STEPS; s++) tv = l16 == s ? tot[s] : tv;
        const float sc = rsqrt_exact(tv / 128 + eps);
        float scale[STEPS];
        static_assert(STEPS <= 5, "the broadcasts below are written out for at most five steps");
        scale[0] = row_lane_bcast<0>(sc);
        if (STEPS > 1) scale[1 % STEPS] = row_lane_bcast<1>(sc);
        if (STEPS > 2) scale[2 % STEPS] = row_lane_bcast<2>(sc);
        if (STEPS > 3) scale[3 % STEPS] = row_lane_bcast<3>(sc);
        if (STEPS > 4) scale[4 % STEPS] = row_lane_bcast<4>(sc);
        // phase 3: scale, rotate, convert, store
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const int h0 = 16 * s + 4 * wave;                               // wave-uniform
            if (F32IN && h0 >= items) break;
            float x[8];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                if (F32IN) { const uint32_t b0 = xin[ti][s][0][p], b1 = xin[ti][s][NW - 1][p]; x[p] = __builtin_bit_cast(float, b0); x[4 + p] = __builtin_bit_cast(float, b1); }
                else { const uint32_t b = xin[ti][s][0][p]; x[2 * p] = __builtin_bit_cast(float, b << 16); x[2 * p + 1] = __builtin_bit_cast(float, b & 0xffff0000u); }
            }
            u32x4 out;
            if constexpr (Q8) {                                             // the Q8 rows, as in qk_rope_wide_tokens (a wave's four heads are of one kind)
                const bool q_heads = h0 < a.nh, v_heads = h0 >= nqk;
                const int h = h0 + hq;
                uint8_t * cwb = (uint8_t *)a.cache + rowi * (2 * (M / 32) * 34);
                float v8[8];
                if (v_heads) {
#pragma unroll
                    for (int k = 0; k < 8; k++) v8[k] = f16r(x[k]);
                } else {
                    const float * wp = nrm + (q_heads ? 0 : 128) + 8 * l16;
                    const f32x4 w0 = *(const f32x4 *)wp, w1 = *(const f32x4 *)(wp + 4);
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const float y1 = (scale[s] * x[k]) * (k < 4 ? w0[k] : w1[k - 4]);
                        v8[k] = f16r(__builtin_fmaf(y1, k < 4 ? c4[0][k] : c4[1][k - 4], mul_ror8(y1, k < 4 ? s4[0][k] : s4[1][k - 4])));
                    }
                    hadamard128_w8(v8, l16);
                }
                if (q_heads) {
#pragma unroll
                    for (int p = 0; p < 4; p++) out[p] = pack_f16x2(v8[2 * p], v8[2 * p + 1]);
                    RSTORE((u32x4 *)(qw + (size_t)h * 128 + 8 * l16), out);
                } else {
                    const size_t b = v_heads ? M / 32 + (size_t)(h - nqk) * 4 + (l16 >> 2) : (size_t)(h - a.nh) * 4 + (l16 >> 2);
                    kv_q8_emit_w8(v8, cwb + b * 34, l16 & 3, a.err, span);
                }
                continue;
            }
            if (h0 >= nqk) {                                                // V heads: fp16 copy
#pragma unroll
                for (int p = 0; p < 4; p++) out[p] = pack_f16x2(x[2 * p], x[2 * p + 1]);
                if (!GEN || span) RSTORE((u32x4 *)(cw + M + (size_t)(h0 - nqk) * 128 + lo), out);
                continue;
            }
            const bool isq = h0 < a.nh;
            const float * wp = nrm + (isq ? 0 : 128) + 8 * l16;
            const f32x4 w0 = *(const f32x4 *)wp, w1 = *(const f32x4 *)(wp + 4);
            float y[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float y1 = (scale[s] * x[k]) * (k < 4 ? w0[k] : w1[k - 4]);
                y[k] = __builtin_fmaf(y1, k < 4 ? c4[0][k] : c4[1][k - 4], mul_ror8(y1, k < 4 ? s4[0][k] : s4[1][k - 4]));
            }
#pragma unroll
            for (int p = 0; p < 4; p++) out[p] = pack_f16x2(y[2 * p], y[2 * p + 1]);
            if (!GEN || isq || span) RSTORE((u32x4 *)((isq ? qw + (size_t)h0 * 128 : cw + (size_t)(h0 - a.nh) * 128) + lo), out);
        }
    }
}
// fp32 rows: any number of heads up to 48 with nh and nkv multiples of 4
template <bool YARN, int TPW, bool Q8>
static bool rope_chunk_launch_f32(const RopeArgs & a, hipStream_t st) {
    const int items = a.nh + 2 * a.nkv;
    if (items > 48 || (a.nh & 3) || (a.nkv & 3)) return false;
    const dim3 grid((a.n + TPW - 1) / TPW), block(256);
    if (a.pos || a.posb || a.page_table || a.rows != 0) {                   // a batch of sequences, each at its own position and row
        switch ((items + 15) >> 4) {
        case 1: qk_rope_chunk<YARN, 1, TPW, true, Q8, true><<<grid, block, 0, st>>>(a); break;
        case 2: qk_rope_chunk<YARN, 2, TPW, true, Q8, true><<<grid, block, 0, st>>>(a); break;
        default: qk_rope_chunk<YARN, 3, TPW, true, Q8, true><<<grid, block, 0, st>>>(a); break;
        }
        return true;
    }
    switch ((items + 15) >> 4) {
    case 1: qk_rope_chunk<YARN, 1, TPW, true, Q8><<<grid, block, 0, st>>>(a); break;
    case 2: qk_rope_chunk<YARN, 2, TPW, true, Q8><<<grid, block, 0, st>>>(a); break;
    default: qk_rope_chunk<YARN, 3, TPW, true, Q8><<<grid, block, 0, st>>>(a); break;
    }
    return true;
}
template <bool YARN, int TPW>
static bool rope_chunk_launch(const RopeArgs & a, hipStream_t st) {
    const int items = a.nh + 2 * a.nkv;
    if (a.pos || a.posb || a.page_table || (items & 15) || items > 80 || (a.nh & 3) || (a.nkv & 3)) return false;
    const dim3 grid((a.n + TPW - 1) / TPW), block(256);
    switch (items >> 4) {
    case 1: qk_rope_chunk<YARN, 1, TPW><<<grid, block, 0, st>>>(a); break;
    case 2: qk_rope_chunk<YARN, 2, TPW><<<grid, block, 0, st>>>(a); break;
    case 3: qk_rope_chunk<YARN, 3, TPW><<<grid, block, 0, st>>>(a); break;
    case 4: qk_rope_chunk<YARN, 4, TPW><<<grid, block, 0, st>>>(a); break;
    default: qk_rope_chunk<YARN, 5, TPW><<<grid, block, 0, st>>>(a); break;
    }
    return true;
}

// ---- pf_qk_nr: any head dim D <= 512, rotary on the first n_rot dims, input heads at head_stride ------------------------------
struct NrArgs {
    const void * x; int head_stride, heads; const float * w; int D, nrot; float theta_scale, eps; int pos0; const int32_t * pos; void * out; int T;
    const int32_t * posb;            // the tape's device-resident position: row r sits at posb[0] + r (pos and pos0 unused)
    const void * x2; int head_stride2, heads2; const float * w2; void * out2;   // a second group of heads per token (k beside q); qk_nr_heads only
    const float * v; int ldv; void * cache; int rows; int * err;                // qk_nr_heads<.., KV>: the token's v row and the cache that takes k and v
};
CAMX_DEV int nr_posi(const NrArgs & a, int tok) { return a.pos ? a.pos[tok] : (a.posb ? a.posb[0] : a.pos0) + tok; }
CAMX_DEV float nr_pos(const NrArgs & a, int tok) { return (float)nr_posi(a, tok); }
// One wave per (token, head), four per workgroup, nothing shared between them: each wave issues its head's loads, computes
// the token's cos / sin for the rotated pairs into its own LDS rows while they are in flight, normalizes, parks the normed
// head in LDS for the partner reads of the rotation, and stores. No barrier; a verify batch of 16 tokens x 28 heads is 448
// independent waves instead of 16 workgroups that loop over their heads.
// KV 1 / 2 (fp32, VEC): the tape's OP_KV_APPEND behind the k heads' OP_QK_NR in the same launch. Each token has heads2 more waves, one per
// head of its v row; the k heads' results and the v heads go to cache row position(token) as OP_KV_APPEND writes them from the fp32
// buffers (1: fp16 [K | V], kv_append16_k; 2: ggml q8_0 blocks, K's then V's, pf_kv_append_rows: a lane's 4 values and its 8-lane group
// are one block's), out2 only if given. A position outside [0, rows): err bit 1, the cache row is not written, the fp32 outputs are.
template <bool BF16, bool VEC, int KV = 0>
__global__ void __launch_bounds__(256) qk_nr_heads(NrArgs a) {
    __shared__ float rc[4][256], rs[4][256];
    __shared__ __attribute__((aligned(16))) float nrm[4][512];
    const int tid = threadIdx.x, lraw = tid & 63, lane = slot_of(lraw), wave = tid >> 6, half = a.nrot / 2;
    const long gw = (long)blockIdx.x * 4 + wave;
    const int hpt = a.heads + a.heads2 + (KV ? a.heads2 : 0);    // heads per token over the groups
    if (gw >= (long)a.T * hpt) return;
    const int tok = (int)(gw / hpt), hh = (int)(gw - (long)tok * hpt);
    [[maybe_unused]] bool row_ok = true;
    [[maybe_unused]] size_t M = 0;
    if constexpr (KV != 0) {
        const long p = nr_posi(a, tok);
        row_ok = p >= 0 && p < a.rows;
        M = (size_t)a.heads2 * a.D;
        if (hh >= a.heads + a.heads2) {                           // (wave-uniform) a head of the token's v row: no arithmetic but the cache's
            const int hv = hh - a.heads - a.heads2;
            if (!row_ok) { if (hv == 0 && lraw == 0) atomicOr(a.err, 1); return; }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int i0 = 256 * j + 4 * lane;
                const bool in = i0 < a.D;
                f32x4 vv = {0.0f, 0.0f, 0.0f, 0.0f};
                if (in) vv = *(const f32x4 *)(a.v + (size_t)tok * a.ldv + (size_t)hv * a.D + i0);
                const size_t e = M + (size_t)hv * a.D + i0;      // the value's index in the cache row's [K | V]
                if (KV == 1) { if (in) *(u32x2 *)((uint16_t *)a.cache + (size_t)p * 2 * M + e) = pack_f16x4(vv); }
                else if (256 * j < a.D) pf_q8_0_emit(vv, (uint8_t *)a.cache + ((size_t)p * (2 * M / 32) + (in ? e / 32 : 0)) * 34, lane & 7, in);
            }
            return;
        }
    }
    const bool g2 = hh >= a.heads;                               // (wave-uniform) this head belongs to the second group
    if (g2) { a.x = a.x2; a.w = a.w2; a.out = a.out2; a.head_stride = a.head_stride2; }
    const size_t hi = g2 ? (size_t)tok * a.heads2 + (hh - a.heads) : (size_t)tok * a.heads + hh;
    const size_t xo = hi * a.head_stride, yo = hi * a.D;
    float xv[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int i0 = 256 * j + 4 * lane;
        if (VEC) {                                               // D, head_stride multiples of 4, aligned bases: i0 .. i0 + 3 are in or out together
            f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (i0 < a.D) v = BF16 ? unpack_bf16x4(*(const u32x2 *)((const uint16_t *)a.x + xo + i0)) : *(const f32x4 *)((const float *)a.x + xo + i0);
            xv[j][0] = v.x; xv[j][1] = v.y; xv[j][2] = v.z; xv[j][3] = v.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = i0 + k;
                xv[j][k] = 0.0f;
                if (i < a.D) xv[j][k] = BF16 ? bf2f(((const uint16_t *)a.x)[xo + i]) : ((const float *)a.x)[xo + i];
            }
        }
    }
    float wv[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int k = 0; k < 4; k++) { const int i = 256 * j + 4 * lane + k; wv[j][k] = i < a.D ? a.w[i] : 0.0f; }
    const float pos = nr_pos(a, tok);
    for (int j = lraw; j < half; j += 64) {
        const float theta = pos * rope_freq(a.theta_scale, j);
        rc[wave][j] = cosf(theta); rs[wave][j] = sinf(theta);
    }
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 2; j++) {
        ss.x = __builtin_fmaf(xv[j][0], xv[j][0], ss.x); ss.y = __builtin_fmaf(xv[j][1], xv[j][1], ss.y);
        ss.z = __builtin_fmaf(xv[j][2], xv[j][2], ss.z); ss.w = __builtin_fmaf(xv[j][3], xv[j][3], ss.w);
    }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)a.D + a.eps);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = 256 * j + 4 * lane + k;
            if (i < a.D) { xv[j][k] = (scale * xv[j][k]) * wv[j][k]; nrm[wave][i] = xv[j][k]; }
        }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): this wave's LDS stores have landed before its reads
#pragma unroll
    for (int j = 0; j < 2; j++) {
        float y[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = 256 * j + 4 * lane + k;
            y[k] = xv[j][k];
            if (i < a.D && i < a.nrot) {
                const int jj = i < half ? i : i - half;
                const float c = rc[wave][jj], sn = rs[wave][jj];
                const float x0 = nrm[wave][jj], x1 = nrm[wave][jj + half];
                y[k] = i < half ? x0 * c - x1 * sn : x0 * sn + x1 * c;
            }
        }
        const int i0 = 256 * j + 4 * lane;
        if constexpr (KV != 0) {
            if (g2) {                                            // a k head: the cache row's K part (and the fp32 buffer only if the caller keeps one)
                const bool in = i0 < a.D;
                const f32x4 v = {y[0], y[1], y[2], y[3]};
                if (in && a.out) *(f32x4 *)((float *)a.out + yo + i0) = v;
                if (!row_ok) continue;                           // (the token's first v wave reports it)
                const long p = nr_posi(a, tok);
                const size_t e = (size_t)(hh - a.heads) * a.D + i0;
                if (KV == 1) { if (in) *(u32x2 *)((uint16_t *)a.cache + (size_t)p * 2 * M + e) = pack_f16x4(v); }
                else if (256 * j < a.D) pf_q8_0_emit(v, (uint8_t *)a.cache + ((size_t)p * (2 * M / 32) + (in ? e / 32 : 0)) * 34, lane & 7, in);
                continue;
            }
        }
        if (VEC) {
            if (i0 < a.D) {
                const f32x4 v = {y[0], y[1], y[2], y[3]};
                if (BF16) *(u32x2 *)((uint16_t *)a.out + yo + i0) = pack_bf16x4_rne(v); else *(f32x4 *)((float *)a.out + yo + i0) = v;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (i0 + k < a.D) { if (BF16) ((uint16_t *)a.out)[yo + i0 + k] = to_bf16(y[k]); else ((float *)a.out)[yo + i0 + k] = y[k]; }
        }
    }
}

// Prefill-sized batches: one workgroup per token, the token's cos / sin computed once (not once per head), each wave walks
// heads wave, wave + 4, .. with the next head's 128-bit loads in flight during the current head's arithmetic.
template <bool BF16>
__global__ void __launch_bounds__(256) qk_nr_tokens_vec(NrArgs a) {
    __shared__ float rc[256], rs[256];
    __shared__ __attribute__((aligned(16))) float nrm[4][512];
    const int tok = blockIdx.x, tid = threadIdx.x, lane = slot_of(tid & 63), wave = tid >> 6, half = a.nrot / 2;
    auto load = [&](float (&xv)[2][4], int h) {
        const size_t xo = ((size_t)tok * a.heads + (h < a.heads ? h : 0)) * a.head_stride;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i0 = 256 * j + 4 * lane;
            f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (i0 < a.D) v = BF16 ? unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)((const uint16_t *)a.x + xo + i0)))
                                   : __builtin_nontemporal_load((const f32x4 *)((const float *)a.x + xo + i0));
            xv[j][0] = v.x; xv[j][1] = v.y; xv[j][2] = v.z; xv[j][3] = v.w;
        }
    };
    float xv[2][4], xn[2][4];
    load(xv, wave);
    float wv[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int k = 0; k < 4; k++) { const int i = 256 * j + 4 * lane + k; wv[j][k] = i < a.D ? a.w[i] : 0.0f; }
    const float pos = nr_pos(a, tok);
    for (int j = tid; j < half; j += 256) {
        const float theta = pos * rope_freq(a.theta_scale, j);
        rc[j] = cosf(theta); rs[j] = sinf(theta);
    }
    __syncthreads();
    for (int h = wave; h < a.heads; h += 4) {
        load(xn, h + 4);
        const size_t yo = ((size_t)tok * a.heads + h) * a.D;
        f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            ss.x = __builtin_fmaf(xv[j][0], xv[j][0], ss.x); ss.y = __builtin_fmaf(xv[j][1], xv[j][1], ss.y);
            ss.z = __builtin_fmaf(xv[j][2], xv[j][2], ss.z); ss.w = __builtin_fmaf(xv[j][3], xv[j][3], ss.w);
        }
        const float tot = wave_groups_in_order(group32_sum(ss));
        const float scale = rsqrt_exact(tot / (float)a.D + a.eps);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i0 = 256 * j + 4 * lane;
#pragma unroll
            for (int k = 0; k < 4; k++) xv[j][k] = (scale * xv[j][k]) * wv[j][k];
            if (i0 < a.D) *(f32x4 *)(nrm[wave] + i0) = (f32x4){xv[j][0], xv[j][1], xv[j][2], xv[j][3]};
        }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): this wave's LDS stores have landed before its reads
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i0 = 256 * j + 4 * lane;
            float y[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = i0 + k;
                y[k] = xv[j][k];
                if (i < a.D && i < a.nrot) {
                    const int jj = i < half ? i : i - half;
                    const float c = rc[jj], sn = rs[jj];
                    const float x0 = nrm[wave][jj], x1 = nrm[wave][jj + half];
                    y[k] = i < half ? x0 * c - x1 * sn : x0 * sn + x1 * c;
                }
            }
            if (i0 < a.D) {
                const f32x4 v = {y[0], y[1], y[2], y[3]};
                if (BF16) *(u32x2 *)((uint16_t *)a.out + yo + i0) = pack_bf16x4_rne(v); else *(f32x4 *)((float *)a.out + yo + i0) = v;
            }
        }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);          // the reads above are done before the next head overwrites the row
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int k = 0; k < 4; k++) xv[j][k] = xn[j][k];
    }
}

// Prefill-sized batches of heads of at most 256 dims whose rotated width is a power of two (8 .. 256): the partner of
// element i (i + nrot / 2 or i - nrot / 2) sits nrot / 8 lanes away, so the rotation is a lane exchange and nothing goes
// through LDS but the token's cos / sin row. Lane p holds dims 4p .. 4p + 3; sin carries the sign of its half. A wave walks
// heads wave, wave + 4, ..; two heads ahead are in flight.
template <int XL> CAMX_DEV float nr_partner(float v) {
    if (XL == 1) return lane_xor1(v);
    if (XL == 2) return lane_xor2(v);
    if (XL == 4) return lane_xor4(v);
    if (XL == 8) return lane_xor8(v);
    if (XL == 16) return lane_xor16(v);
    return __shfl_xor(v, 32, 64);
}
template <bool BF16, int XL>
__global__ void __launch_bounds__(256) qk_nr_tokens_fast(NrArgs a) {
    __shared__ __attribute__((aligned(16))) float rc[128], rs[128];
    typedef typename std::conditional<BF16, u32x2, f32x4>::type Raw;
    const int tok = blockIdx.x, tid = threadIdx.x, lane = slot_of(tid & 63), wave = tid >> 6, nrot = 8 * XL, half = nrot / 2;
    const int i0 = 4 * lane;
    const bool on = i0 < a.D, rot = i0 < nrot;
    auto load = [&](int h) {
        Raw v = {};
        if (h < a.heads && on) {
            const size_t xo = ((size_t)tok * a.heads + h) * a.head_stride + i0;
            if constexpr (BF16) v = __builtin_nontemporal_load((const u32x2 *)((const uint16_t *)a.x + xo));
            else v = __builtin_nontemporal_load((const f32x4 *)((const float *)a.x + xo));
        }
        return v;
    };
    Raw r0 = load(wave), r1 = load(wave + 4);
    f32x4 wv = {0.0f, 0.0f, 0.0f, 0.0f};
    if (on) wv = *(const f32x4 *)(a.w + i0);
    const float pos = nr_pos(a, tok);
    if (tid < half) {
        const float theta = pos * rope_freq(a.theta_scale, tid);
        rc[tid] = cosf(theta); rs[tid] = sinf(theta);
    }
    __syncthreads();
    f32x4 c4 = {1.0f, 1.0f, 1.0f, 1.0f}, s4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (rot) {
        const int jj = i0 & (half - 1);
        c4 = *(const f32x4 *)(rc + jj); s4 = *(const f32x4 *)(rs + jj);
        if (i0 < half) { s4.x = -s4.x; s4.y = -s4.y; s4.z = -s4.z; s4.w = -s4.w; }
    }
    for (int h = wave; h < a.heads; h += 8) {
        const Raw n0 = load(h + 8), n1 = load(h + 12);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int hh = h + 4 * u;
            if (hh < a.heads) {                                 // uniform per wave
                const Raw raw = u ? r1 : r0;
                f32x4 x;
                if constexpr (BF16) x = unpack_bf16x4(raw); else x = raw;
                f32x4 ss;
                ss.x = __builtin_fmaf(x.x, x.x, 0.0f); ss.y = __builtin_fmaf(x.y, x.y, 0.0f); ss.z = __builtin_fmaf(x.z, x.z, 0.0f); ss.w = __builtin_fmaf(x.w, x.w, 0.0f);
                const float tot = wave_groups_in_order(group32_sum(ss));
                const float scale = rsqrt_exact(tot / (float)a.D + a.eps);
                x.x = (scale * x.x) * wv.x; x.y = (scale * x.y) * wv.y; x.z = (scale * x.z) * wv.z; x.w = (scale * x.w) * wv.w;
                f32x4 pr;
                pr.x = nr_partner<XL>(x.x); pr.y = nr_partner<XL>(x.y); pr.z = nr_partner<XL>(x.z); pr.w = nr_partner<XL>(x.w);
                f32x4 y = x;
                if (rot) { y.x = x.x * c4.x + pr.x * s4.x; y.y = x.y * c4.y + pr.y * s4.y; y.z = x.z * c4.z + pr.z * s4.z; y.w = x.w * c4.w + pr.w * s4.w; }
                if (on) {
                    const size_t yo = ((size_t)tok * a.heads + hh) * a.D + i0;
                    if (BF16) *(u32x2 *)((uint16_t *)a.out + yo) = pack_bf16x4_rne(y); else *(f32x4 *)((float *)a.out + yo) = y;
                }
            }
        }
        r0 = n0; r1 = n1;
    }
}

// Heads of exactly 256 dims at prefill sizes: 32 lanes per head (lane l holds dims 8 l .. 8 l + 7), two heads per wave
// instruction, NS wave steps (2 NS heads) per wave with all their loads issued first and ONE IEEE sqrt + divide for all of them
// (lane s of a half-wave takes step s). The 32-thread butterfly of the norm sum is lane ^ 2, lane ^ 1 and three in-register
// levels (the pairs and order of thread xor 16, 8, 4, 2, 1); the eight group sums are fetched by swizzles and added in order.
// The rotary partner (dim i +- nrot / 2) sits XL = nrot / 16 lanes away.
template <int J> CAMX_DEV float swz_group32(float v) {       // every lane of a 32-lane half reads the half's lane 4 J + (lane & 3)
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x03 | ((4 * J) << 5)));
}
template <int S> CAMX_DEV float half32_lane_bcast(float v) { // every lane of a 32-lane half reads the half's lane S
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x00 | (S << 5)));
}
template <int XL> CAMX_DEV float nr8_partner(float v) {
    if (XL == 1) return dpp_xor1(v);
    if (XL == 2) return dpp_xor2(v);
    if (XL == 4) return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x101F));
    if (XL == 8) return dpp_ror8(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
template <bool BF16, int XL, int NS>
__global__ void __launch_bounds__(256) qk_nr_tokens_w8(NrArgs a) {
    __shared__ __attribute__((aligned(16))) float rc[128], rs[128];
    constexpr int NW = BF16 ? 1 : 2;
    const int tok = blockIdx.x, tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, hf = lane >> 5, wave = tid >> 6;
    const int nrot = 16 * XL, half = nrot / 2, i0 = 8 * l32;
    const bool rot = i0 < nrot;
    const int per_pass = 8 * NS;                                        // heads per workgroup pass: wave w, step s, half hf -> head 8 s + 2 w + hf
    u32x4 raw[NS][NW];
    auto load = [&](int base) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const int h = base + 8 * s + 2 * wave + hf;
#pragma unroll
            for (int w = 0; w < NW; w++) raw[s][w] = (u32x4){0u, 0u, 0u, 0u};
            if (h < a.heads) {
                const size_t xo = ((size_t)tok * a.heads + h) * a.head_stride + i0;
                if (BF16) raw[s][0] = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)a.x + xo));
                else { raw[s][0] = __builtin_nontemporal_load((const u32x4 *)((const float *)a.x + xo)); raw[s][NW - 1] = __builtin_nontemporal_load((const u32x4 *)((const float *)a.x + xo + 4)); }
            }
        }
    };
    load(0);
    const f32x4 w0 = *(const f32x4 *)(a.w + i0), w1 = *(const f32x4 *)(a.w + i0 + 4);
    const float pos = nr_pos(a, tok);
    if (tid < half) {
        const float theta = pos * rope_freq(a.theta_scale, tid);
        rc[tid] = cosf(theta); rs[tid] = sinf(theta);
    }
    __syncthreads();
    f32x4 c4[2] = {{1.0f, 1.0f, 1.0f, 1.0f}, {1.0f, 1.0f, 1.0f, 1.0f}}, s4[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
    if (rot) {
        const int jj = i0 & (half - 1);
        c4[0] = *(const f32x4 *)(rc + jj); c4[1] = *(const f32x4 *)(rc + jj + 4);
        s4[0] = *(const f32x4 *)(rs + jj); s4[1] = *(const f32x4 *)(rs + jj + 4);
        if (i0 < half) { s4[0] = -s4[0]; s4[1] = -s4[1]; }              // dims below nrot / 2 take -(partner * sin)
    }
    for (int base = 0; base < a.heads; base += per_pass) {
        float x[NS][8], tot[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) {
            if (BF16) {
#pragma unroll
                for (int p = 0; p < 4; p++) { const uint32_t b = raw[s][0][p]; x[s][2 * p] = __builtin_bit_cast(float, b << 16); x[s][2 * p + 1] = __builtin_bit_cast(float, b & 0xffff0000u); }
            } else {
#pragma unroll
                for (int p = 0; p < 4; p++) { const uint32_t b0 = raw[s][0][p], b1 = raw[s][NW - 1][p]; x[s][p] = __builtin_bit_cast(float, b0); x[s][4 + p] = __builtin_bit_cast(float, b1); }
            }
            float sq[8];
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = x[s][k] * x[s][k];
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor2(sq[k]);            // thread ^ 16
#pragma unroll
            for (int k = 0; k < 8; k++) sq[k] = add_xor1(sq[k]);            // thread ^ 8
            const float b0 = sq[0] + sq[4], b1 = sq[1] + sq[5], b2 = sq[2] + sq[6], b3 = sq[3] + sq[7];   // thread ^ 4
            const float e0 = b0 + b2, e1 = b1 + b3;                         // thread ^ 2
            const float g = e0 + e1;                                        // thread ^ 1
            tot[s] = ((((((swz_group32<0>(g) + swz_group32<1>(g)) + swz_group32<2>(g)) + swz_group32<3>(g)) + swz_group32<4>(g)) + swz_group32<5>(g)) +
                      swz_group32<6>(g)) + swz_group32<7>(g);
        }
        if (base + per_pass < a.heads) load(base + per_pass);               // the next pass's rows, in flight during this pass's arithmetic
        float tv = tot[0];
#pragma unroll
        for (int s = 1; s < NS; s++) tv = l32 == s ? tot[s] : tv;
        const float sc = rsqrt_exact(tv / 256.0f + a.eps);
        float scale[NS];
        static_assert(NS <= 4, "the broadcasts below are written out for at most four steps");
        scale[0] = half32_lane_bcast<0>(sc);
        if (NS > 1) scale[1 % NS] = half32_lane_bcast<1>(sc);
        if (NS > 2) scale[2 % NS] = half32_lane_bcast<2>(sc);
        if (NS > 3) scale[3 % NS] = half32_lane_bcast<3>(sc);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            if (base + 8 * s + 2 * wave >= a.heads) break;                  // wave-uniform: neither half has a head
            const int h = base + 8 * s + 2 * wave + hf;
            float y[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float xn = (scale[s] * x[s][k]) * (k < 4 ? w0[k] : w1[k - 4]);
                const float pr = nr8_partner<XL>(xn);
                y[k] = rot ? xn * (k < 4 ? c4[0][k] : c4[1][k - 4]) + pr * (k < 4 ? s4[0][k] : s4[1][k - 4]) : xn;
            }
            if (h < a.heads) {
                const size_t yo = ((size_t)tok * a.heads + h) * 256 + i0;
                if (BF16) {
                    const u32x2 lo = pack_bf16x4_rne((f32x4){y[0], y[1], y[2], y[3]}), hi = pack_bf16x4_rne((f32x4){y[4], y[5], y[6], y[7]});
                    __builtin_nontemporal_store((u32x4){lo.x, lo.y, hi.x, hi.y}, (u32x4 *)((uint16_t *)a.out + yo));
                } else {
                    __builtin_nontemporal_store((f32x4){y[0], y[1], y[2], y[3]}, (f32x4 *)((float *)a.out + yo));
                    __builtin_nontemporal_store((f32x4){y[4], y[5], y[6], y[7]}, (f32x4 *)((float *)a.out + yo + 4));
                }
            }
        }
    }
}

static void launch_nr(const NrArgs & a, int io, hipStream_t st) {
    const int es = io ? 2 : 4;
    const bool vec = (a.D & 3) == 0 && (a.head_stride & 3) == 0 && ((uintptr_t)a.x & (4 * es - 1)) == 0 && ((uintptr_t)a.out & (4 * es - 1)) == 0;
    const bool vec8 = (a.head_stride & 7) == 0 && ((uintptr_t)a.x & 15) == 0 && ((uintptr_t)a.out & 15) == 0 && ((uintptr_t)a.w & 15) == 0;
    if (vec8 && a.D == 256 && a.heads >= 8 && (long)a.T * a.heads >= 4096 && a.nrot >= 16 && (a.nrot & (a.nrot - 1)) == 0) {
#define NR_W8(XL) (io ? qk_nr_tokens_w8<true, XL, 3><<<dim3(a.T), dim3(256), 0, st>>>(a) : qk_nr_tokens_w8<false, XL, 3><<<dim3(a.T), dim3(256), 0, st>>>(a))
        switch (a.nrot) { case 16: NR_W8(1); break; case 32: NR_W8(2); break; case 64: NR_W8(4); break; case 128: NR_W8(8); break; default: NR_W8(16); break; }
#undef NR_W8
        return;
    }
    if (vec && a.heads >= 8 && (long)a.T * a.heads >= 4096 && a.D <= 256 && a.nrot >= 8 && a.nrot <= a.D && (a.nrot & (a.nrot - 1)) == 0) {
#define NR_FAST(XL) (io ? qk_nr_tokens_fast<true, XL><<<dim3(a.T), dim3(256), 0, st>>>(a) : qk_nr_tokens_fast<false, XL><<<dim3(a.T), dim3(256), 0, st>>>(a))
        switch (a.nrot) { case 8: NR_FAST(1); break; case 16: NR_FAST(2); break; case 32: NR_FAST(4); break; case 64: NR_FAST(8); break;
                          case 128: NR_FAST(16); break; default: NR_FAST(32); break; }
#undef NR_FAST
        return;
    }
    if (vec && a.heads >= 8 && (long)a.T * a.heads >= 4096) {          // a prefill chunk: share the token's cos / sin among its heads
        if (io) qk_nr_tokens_vec<true><<<dim3(a.T), dim3(256), 0, st>>>(a); else qk_nr_tokens_vec<false><<<dim3(a.T), dim3(256), 0, st>>>(a);
        return;
    }
    const dim3 grid((unsigned)(((long)a.T * a.heads + 3) / 4)), block(256);
    if (io) { if (vec) qk_nr_heads<true, true><<<grid, block, 0, st>>>(a); else qk_nr_heads<true, false><<<grid, block, 0, st>>>(a); }
    else { if (vec) qk_nr_heads<false, true><<<grid, block, 0, st>>>(a); else qk_nr_heads<false, false><<<grid, block, 0, st>>>(a); }
}

// ---- the dense Q8 line's per-token chain in one launch ------------------------------------------------------------------------------
// The reference appends, per full-attention layer, OP_QK_NR (k) -> OP_HADAMARD 256 (k) -> OP_HADAMARD 64 (v) -> OP_KV_APPEND (Q8 blocks with
// the codec's refusal rules) and OP_QK_NR (q) -> OP_HADAMARD 256 (q) (python/caminus/engine/q35_dense.py:409-418; kernels/k3_q35_ops.h:341-364,
// kernels/k3_q35_kvq8_ops.h:16-50, kernels/own_kv_codec.h:57-72): six tape segments through fp32 buffers. Here a half-wave owns one item of
// 256 values (a q head, a k head, or 256 values of the token's v row = four 64-point chunks), lane l at values 8 l .. 8 l + 7: norm and
// rotary as qk_nr_tokens_w8 forms them, the Walsh-Hadamard stages in the reference's order (h = 1, 2, 4 in registers, then lanes l ^ 1,
// 2, 4, 8, 16; 8 lanes per 64-point chunk), the scale 1 / sqrtf(n) (a power of two), and the K / V blocks of 32 values from 4 lanes x 8.
// Sums and differences are the same operations on the same operands as in the separate kernels, so every byte is theirs.
template <int LOGL> CAMX_DEV void hadamard_w8_lanes(float (&e)[8], int l, float scale) {     // 8 << LOGL points: 1 << LOGL lanes x 8 registers
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
        for (int k = 0; k < 8; k++)
            if (!(k & h)) { const float a = e[k], b = e[k + h]; e[k] = a + b; e[k + h] = a - b; }
#define W8L_STAGE(BIT, PARTNER)                                                                                  \
    {                                                                                                              \
        const uint32_t m = (l & BIT) ? 0x80000000u : 0u;                                                           \
        _Pragma("unroll") for (int k = 0; k < 8; k++) {                                                            \
            const float own = e[k];                                                                                \
            e[k] = PARTNER(own) + __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, own) ^ m);                \
        }                                                                                                          \
    }
#define W8L_XOR4(x) __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x101F))
#define W8L_XOR16(x) __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x401F))
    if (LOGL > 0) W8L_STAGE(1, dpp_full<0xB1>)
    if (LOGL > 1) W8L_STAGE(2, dpp_full<0x4E>)
    if (LOGL > 2) W8L_STAGE(4, W8L_XOR4)
    if (LOGL > 3) W8L_STAGE(8, dpp_full<0x128>)
    if (LOGL > 4) W8L_STAGE(16, W8L_XOR16)
#undef W8L_XOR16
#undef W8L_XOR4
#undef W8L_STAGE
#pragma unroll
    for (int k = 0; k < 8; k++) e[k] *= scale;
}
struct NrQ8Args {
    const float * q; int q_stride, nh; const float * k; int ldk; const float * v; int ldv; int nkv;
    const float * qn, * kn; float theta_scale, eps; int pos0; const int32_t * posb, * pos;
    float * qo; uint8_t * cache; int rows; int * err; int T;
};
template <int XL>
__global__ void __launch_bounds__(256) qk_nr_q8_k(NrQ8Args a) {
    __shared__ __attribute__((aligned(16))) float rc[128], rs[128];
    constexpr int nrot = 16 * XL, half = nrot / 2;
    const int tid = threadIdx.x, l32 = tid & 31, hw = tid >> 5, i0 = 8 * l32;
    const int items = a.nh + 2 * a.nkv, G = (items + 7) >> 3;
    const int tok = blockIdx.x / G, item = (blockIdx.x - tok * G) * 8 + hw;
    const bool on = item < items;
    const int kind = !on ? 3 : item < a.nh ? 0 : item < a.nh + a.nkv ? 1 : 2;                 // q head, k head, 256 values of v
    const float * src = kind == 1 ? a.k + (size_t)tok * a.ldk + (size_t)(item - a.nh) * 256
                      : kind == 2 ? a.v + (size_t)tok * a.ldv + (size_t)(item - a.nh - a.nkv) * 256
                      : a.q + ((size_t)tok * a.nh + (on ? item : 0)) * a.q_stride;
    const f32x4 r0 = *(const f32x4 *)(src + i0), r1 = *(const f32x4 *)(src + i0 + 4);
    const long pos = (long)(a.pos ? a.pos[tok] : (a.posb ? a.posb[0] : a.pos0)) + (a.pos ? 0 : tok);
    if (tid < half) {
        const float theta = (float)(int)pos * rope_freq(a.theta_scale, tid);
        rc[tid] = cosf(theta); rs[tid] = sinf(theta);
    }
    __syncthreads();
    if (!on) return;
    float e[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
    if (kind < 2) {
        const float * wp = (kind == 0 ? a.qn : a.kn) + i0;
        const f32x4 w0 = *(const f32x4 *)wp, w1 = *(const f32x4 *)(wp + 4);
        float sq[8];
#pragma unroll
        for (int k = 0; k < 8; k++) sq[k] = e[k] * e[k];
#pragma unroll
        for (int k = 0; k < 8; k++) sq[k] = add_xor2(sq[k]);
#pragma unroll
        for (int k = 0; k < 8; k++) sq[k] = add_xor1(sq[k]);
        const float b0 = sq[0] + sq[4], b1 = sq[1] + sq[5], b2 = sq[2] + sq[6], b3 = sq[3] + sq[7];
        const float e0 = b0 + b2, e1 = b1 + b3;
        const float g = e0 + e1;
        const float tot = ((((((swz_group32<0>(g) + swz_group32<1>(g)) + swz_group32<2>(g)) + swz_group32<3>(g)) + swz_group32<4>(g)) + swz_group32<5>(g)) +
                           swz_group32<6>(g)) + swz_group32<7>(g);
        const float scale = rsqrt_exact(tot / 256.0f + a.eps);
        const bool rot = i0 < nrot;
        f32x4 c4[2] = {{1.0f, 1.0f, 1.0f, 1.0f}, {1.0f, 1.0f, 1.0f, 1.0f}}, s4[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
        if (rot) {
            const int jj = i0 & (half - 1);
            c4[0] = *(const f32x4 *)(rc + jj); c4[1] = *(const f32x4 *)(rc + jj + 4);
            s4[0] = *(const f32x4 *)(rs + jj); s4[1] = *(const f32x4 *)(rs + jj + 4);
            if (i0 < half) { s4[0] = -s4[0]; s4[1] = -s4[1]; }
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float xn = (scale * e[k]) * (k < 4 ? w0[k] : w1[k - 4]);
            const float pr = nr8_partner<XL>(xn);
            e[k] = rot ? xn * (k < 4 ? c4[0][k] : c4[1][k - 4]) + pr * (k < 4 ? s4[0][k] : s4[1][k - 4]) : xn;
        }
        hadamard_w8_lanes<5>(e, l32, 0.0625f);
    } else hadamard_w8_lanes<3>(e, l32, 0.125f);
    if (kind == 0) {
        float * o = a.qo + ((size_t)tok * a.nh + item) * 256 + i0;
        *(f32x4 *)o = (f32x4){e[0], e[1], e[2], e[3]}; *(f32x4 *)(o + 4) = (f32x4){e[4], e[5], e[6], e[7]};
        return;
    }
    const bool span = pos >= 0 && pos < a.rows;
    if (!span && l32 == 0) atomicOr(a.err, 1);
    const size_t nb = (size_t)a.nkv * 8;                                                     // blocks of K (and of V) per row
    const size_t b = (kind == 1 ? (size_t)(item - a.nh) * 8 : nb + (size_t)(item - a.nh - a.nkv) * 8) + (l32 >> 2);
    uint8_t * row = a.cache + (size_t)(span ? pos : 0) * (2 * nb * 34);
    kv_q8_emit_w8(e, row + b * 34, l32 & 3, a.err, span);
}

__global__ void rope_freqs_k(float theta_scale, int n, float * out) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < n) out[j] = rope_freq(theta_scale, j);
}

static int rope_check(const RopeArgs & a, bool q8, bool bf16in) {
    if (!a.qkv || !a.par || !a.q16 || !a.cache || a.n < 0 || a.nh < 1 || a.nkv < 1 || a.ldq < (a.nh + 2 * a.nkv) * 128 || (a.ldq & 3)) return CAMX_EINVAL;
    if (((uintptr_t)a.qkv & (bf16in ? 7 : 15)) || ((uintptr_t)a.par & 15) || ((uintptr_t)a.q16 & 7) || ((uintptr_t)a.cache & (q8 ? 1 : 7))) return CAMX_EINVAL;
    if (q8 && !a.err) return CAMX_EINVAL;
    if (a.page_table && (a.page < 1 || a.n_pages < 1 || a.pt_stride < 1 || !a.err)) return CAMX_EINVAL;
    if (!a.pos && !a.posb && (a.pos0 < 0 || a.pos0 > 0x7fffffff - a.n)) return CAMX_EINVAL;     // the reference's host span check (python/caminus/engine/k3.py:413-433)
    if (a.posb && (!a.err || a.rows < 1)) return CAMX_EINVAL;
    return CAMX_OK;
}
template <bool BF16IN, int TPW>
static void rope_dispatch(const RopeArgs & a, int yarn, bool q8, hipStream_t st) {
    if (TPW == 1 && a.n <= 256) {                  // a batch that does not fill the chip: ten waves per token (256 tokens: 4.9 us against 6.0)
        const dim3 grid(a.n), block(640);
        if (q8) { if (yarn) qk_rope_tokens<true, true, BF16IN, 1, 10, 2><<<grid, block, 0, st>>>(a); else qk_rope_tokens<false, true, BF16IN, 1, 10, 2><<<grid, block, 0, st>>>(a); }
        else { if (yarn) qk_rope_tokens<true, false, BF16IN, 1, 10, 2><<<grid, block, 0, st>>>(a); else qk_rope_tokens<false, false, BF16IN, 1, 10, 2><<<grid, block, 0, st>>>(a); }
        return;
    }
    const dim3 grid((a.n + TPW - 1) / TPW), block(256);
    if (q8) { if (yarn) qk_rope_tokens<true, true, BF16IN, TPW><<<grid, block, 0, st>>>(a); else qk_rope_tokens<false, true, BF16IN, TPW><<<grid, block, 0, st>>>(a); }
    else { if (yarn) qk_rope_tokens<true, false, BF16IN, TPW><<<grid, block, 0, st>>>(a); else qk_rope_tokens<false, false, BF16IN, TPW><<<grid, block, 0, st>>>(a); }
}
static int rope_launch(const RopeArgs & a, int yarn, bool q8, hipStream_t st, bool bf16in = false) {
    if (rope_check(a, q8, bf16in)) return CAMX_EINVAL;
    if (a.n == 0) return CAMX_OK;
    const bool aligned = (a.ldq & (bf16in ? 7 : 3)) == 0 && ((uintptr_t)a.qkv & 15) == 0 && ((uintptr_t)a.q16 & 15) == 0 && ((uintptr_t)a.cache & 15) == 0;
    const bool wide = (!q8 || !bf16in) && !a.page_table && aligned;
    // a batch of 2048 and more sequences through a page table: the chunk kernel with the token kernels' addressing and refusals
    if (a.page_table && !bf16in && aligned && a.n >= 2048 &&
        (q8 ? (yarn ? rope_chunk_launch_f32<true, 1, true>(a, st) : rope_chunk_launch_f32<false, 1, true>(a, st))
            : (yarn ? rope_chunk_launch_f32<true, 1, false>(a, st) : rope_chunk_launch_f32<false, 1, false>(a, st)))) CAMX_LAUNCH_RET();
    // one token per workgroup: 29.9 us for 4096 tokens x 80 heads on cold lines (two tokens: 32.4, four: 34.9; the general kernel below: 32.3)
    if (wide && bf16in && a.n >= 2048 && (yarn ? rope_chunk_launch<true, 1>(a, st) : rope_chunk_launch<false, 1>(a, st))) {}
    else if (wide && bf16in && a.n >= 2048) {          // enough tokens to fill the chip two to a workgroup (4096 tokens, every launch on cold lines: 32.2 us; four: 34.0, one: 33.7)
        const dim3 g2((a.n + 1) / 2);
        if (yarn) qk_rope_wide_tokens<true, 2, false, 5, false><<<g2, dim3(256), 0, st>>>(a); else qk_rope_wide_tokens<false, 2, false, 5, false><<<g2, dim3(256), 0, st>>>(a);
    }
    else if (wide && bf16in) { if (yarn) qk_rope_wide_tokens<true, 1, false, 5, false><<<dim3(a.n), dim3(256), 0, st>>>(a); else qk_rope_wide_tokens<false, 1, false, 5, false><<<dim3(a.n), dim3(256), 0, st>>>(a); }
    else if (wide && !q8 && a.n >= 2048 && (yarn ? rope_chunk_launch_f32<true, 1, false>(a, st) : rope_chunk_launch_f32<false, 1, false>(a, st))) {}
    else if (wide && q8 && a.n >= 2048 && (yarn ? rope_chunk_launch_f32<true, 1, true>(a, st) : rope_chunk_launch_f32<false, 1, true>(a, st))) {}
    else if (wide && a.n >= 2048) {               // fp32 rows of a prefill chunk: the same kernel, three wave steps (48 heads) per pass
        const dim3 g4((a.n + 3) / 4);
        if (q8) { if (yarn) qk_rope_wide_tokens<true, 4, true, 3, true><<<g4, dim3(256), 0, st>>>(a); else qk_rope_wide_tokens<false, 4, true, 3, true><<<g4, dim3(256), 0, st>>>(a); }
        else { if (yarn) qk_rope_wide_tokens<true, 4, true, 3, false><<<g4, dim3(256), 0, st>>>(a); else qk_rope_wide_tokens<false, 4, true, 3, false><<<g4, dim3(256), 0, st>>>(a); }
    }
    else if (bf16in) rope_dispatch<true, 1>(a, yarn, q8, st);
    else rope_dispatch<false, 1>(a, yarn, q8, st);
    CAMX_LAUNCH_RET();
}

extern "C" {

// q3p_qk_rope: n tokens at positions pos0 .. pos0 + n - 1; cache = fp16 rows [K | V] indexed by position
int camx_q3p_qk_rope(const float * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint16_t * cache,
                     int n, int yarn, hipStream_t st) {
    RopeArgs a = {qkv, ldq, nh, nkv, par, pos0, nullptr, q16, cache, nullptr, nullptr, 0, 0, 0, n, 0};
    return rope_launch(a, yarn, false, st);
}
// q3p_qk_rope_q8: the Q8 cache rows (K rotated by the 128-point Hadamard transform, V unrotated); err bit 2 on a refused block
int camx_q3p_qk_rope_q8(const float * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint8_t * cache,
                        int * err, int n, int yarn, hipStream_t st) {
    RopeArgs a = {qkv, ldq, nh, nkv, par, pos0, nullptr, q16, cache, err, nullptr, 0, 0, 0, n, 0};
    return rope_launch(a, yarn, true, st);
}
// batched decode form: sequence t at its own position pos[t]; row address through a page table
// (page_table[t * pt_stride + pos / page] * page + pos % page) when page_table is given, else row = pos[t] of a cache of n_pages rows.
// err bit 1: a position outside the sequence's table row (pos < 0 or pos / page >= pt_stride) or outside the unpaged cache;
// err bit 8: a page id outside [0, n_pages). Either way that sequence's row is not written. q8 = 0 writes fp16 rows.
int camx_qk_rope_paged(const float * qkv, int ldq, int nh, int nkv, const float * par, const int32_t * pos, uint16_t * q16, void * cache,
                       int * err, const int32_t * page_table, int pt_stride, int page, int n_pages, int n, int yarn, int q8, hipStream_t st) {
    if (!pos || !err || (!page_table && n_pages < 1)) return CAMX_EINVAL;
    RopeArgs a = {qkv, ldq, nh, nkv, par, 0, pos, q16, cache, err, page_table, pt_stride, page, n_pages, n, page_table ? 0 : n_pages};
    return rope_launch(a, yarn, q8 != 0, st);
}

// q3p_qk_rope on bf16 activations: qkv bf16 [n][ldq] widened exactly, then the same statements (a dense bf16 prefill chunk)
int camx_qk_rope_bf16(const uint16_t * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint16_t * cache,
                      int n, int yarn, hipStream_t st) {
    RopeArgs a = {qkv, ldq, nh, nkv, par, pos0, nullptr, q16, cache, nullptr, nullptr, 0, 0, 0, n, 0};
    return rope_launch(a, yarn, false, st, true);
}

// pf_qk_nr: out [T][heads][D] = rotary(rms_norm(x head) * w) at position pos0 + row; io 0 fp32, 1 bf16 in / out
int camx_pf_qk_nr(const void * xin, int head_stride, int heads, const float * w, int D, int nrot, float theta_scale, float eps, int pos0,
                  void * out, int T, int io, hipStream_t st) {
    if (!xin || !w || !out || T < 0 || heads < 1 || D < 1 || D > 512 || head_stride < D || nrot < 0 || nrot > D || (nrot & 1) || io < 0 || io > 1) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    NrArgs a = {xin, head_stride, heads, w, D, nrot, theta_scale, eps, pos0, nullptr, out, T};
    launch_nr(a, io, st);
    CAMX_LAUNCH_RET();
}
// the same with one position per row (a speculative-verify batch)
int camx_qk_nr_pos(const void * xin, int head_stride, int heads, const float * w, int D, int nrot, float theta_scale, float eps,
                   const int32_t * pos, void * out, int T, int io, hipStream_t st) {
    if (!xin || !w || !out || !pos || T < 0 || heads < 1 || D < 1 || D > 512 || head_stride < D || nrot < 0 || nrot > D || (nrot & 1) || io < 0 || io > 1) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    NrArgs a = {xin, head_stride, heads, w, D, nrot, theta_scale, eps, 0, pos, out, T};
    launch_nr(a, io, st);
    CAMX_LAUNCH_RET();
}
// OP_QK_NR by its Seg fields (python/caminus/engine/k3.py:1057-1063): a = x, pad1 = head_stride, W = w, asum = pos (int32 [1] on the device:
// row r sits at pos[0] + r / heads), y = out, out_f32 = n_rot, rs = theta_scale, pad2 = the bit pattern of eps, N = T * heads, K = dim; fp32
int camx_op_qk_nr(const float * x, int head_stride, int heads, int dim, const float * w, const int32_t * pos, float * out, int n_rot, float theta_scale,
                  int eps_bits, int T, hipStream_t st) {
    if (!x || !w || !out || !pos || T < 0 || heads < 1 || dim < 1 || dim > 512 || head_stride < dim || n_rot < 0 || n_rot > dim || (n_rot & 1)) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    NrArgs a = {x, head_stride, heads, w, dim, n_rot, theta_scale, __builtin_bit_cast(float, eps_bits), 0, nullptr, out, T, pos};
    launch_nr(a, 0, st);
    CAMX_LAUNCH_RET();
}
// q and k heads of a token in one launch (two OP_QK_NR segments of the tape, python/caminus/engine/q35_dense.py:408-415): group 1 = nh heads at
// xq + (t * nh + h) * q_stride with weight wq -> outq [T][nh][D]; group 2 = nkv heads at xk + (t * nkv + h) * k_stride with wk -> outk. Row t at
// pos ? pos[t] : (pos_dev ? pos_dev[0] : pos0) + t. A wave per head (the decode / verify form of camx_pf_qk_nr at every size).
int camx_qk_nr_qk(const void * xq, int q_stride, int nh, const float * wq, const void * xk, int k_stride, int nkv, const float * wk, int D, int nrot,
                  float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, void * outq, void * outk, int T, int io, hipStream_t st) {
    if (!xq || !xk || !wq || !wk || !outq || !outk || T < 0 || nh < 1 || nkv < 1 || D < 1 || D > 512 || q_stride < D || k_stride < D || nrot < 0 || nrot > D ||
        (nrot & 1) || io < 0 || io > 1 || (!pos && !pos_dev && (pos0 < 0 || pos0 > 0x7fffffff - T))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if ((long)T * nh >= 12288) {          // a prefill-sized batch: two launches of the kernels that share a token's cos / sin among its heads (2 - 3 times faster there)
        NrArgs aq = {xq, q_stride, nh, wq, D, nrot, theta_scale, eps, pos0, pos, outq, T, pos_dev}, ak = {xk, k_stride, nkv, wk, D, nrot, theta_scale, eps, pos0, pos, outk, T, pos_dev};
        launch_nr(aq, io, st); launch_nr(ak, io, st);
        CAMX_LAUNCH_RET();
    }
    NrArgs a = {xq, q_stride, nh, wq, D, nrot, theta_scale, eps, pos0, pos, outq, T, pos_dev, xk, k_stride, nkv, wk, outk};
    const int es = io ? 2 : 4;
    const bool vec = (D & 3) == 0 && ((q_stride | k_stride) & 3) == 0 && (((uintptr_t)xq | (uintptr_t)xk | (uintptr_t)outq | (uintptr_t)outk) & (4 * es - 1)) == 0;
    const dim3 grid((unsigned)(((long)T * (nh + nkv) + 3) / 4)), block(256);
    if (io) { if (vec) qk_nr_heads<true, true><<<grid, block, 0, st>>>(a); else qk_nr_heads<true, false><<<grid, block, 0, st>>>(a); }
    else { if (vec) qk_nr_heads<false, true><<<grid, block, 0, st>>>(a); else qk_nr_heads<false, false><<<grid, block, 0, st>>>(a); }
    CAMX_LAUNCH_RET();
}
// The fp16 / q8_0 cache lines' three tape segments in one launch: OP_QK_NR (k) -> OP_KV_APPEND and OP_QK_NR (q) (python/caminus/engine/
// q3moe_one.py:316-318, 368-370; python/caminus/engine/q35_dense.py:408-415; kernels/k3_gguf_ops.h:1520-1553). q, k heads and positions as
// camx_qk_nr_qk (fp32); v fp32 [T][nkv * D] at ldv; qo [T][nh][D]; ko [T][nkv][D] optional (NULL: the normed k only reaches the cache);
// cache row position(t): work 0 fp16 [K | V] (8-byte aligned), work 1 ggml q8_0 blocks (D % 32 == 0). err bit 1: a position outside
// [0, rows) (that cache row is not written; qo and ko are). D % 4 == 0, strides % 4 == 0, 16-byte aligned fp32 pointers.
int camx_i_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, const int32_t * posb, int rows, int * err, int T, hipStream_t st);   // pfglue.hip
int camx_i_pf_kv_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, const int32_t * posb, int rows, int * err, int T, hipStream_t st);    // kv.hip
int camx_qk_nr_kv(const float * q, int q_stride, int nh, const float * wq, const float * k, int k_stride, const float * v, int ldv, int nkv, const float * wk,
                  int D, int nrot, float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, float * qo, float * ko, void * cache,
                  int work, int rows, int * err, int T, hipStream_t st) {
    if (!q || !k || !v || !wq || !wk || !qo || !cache || !err || T < 0 || nh < 1 || nkv < 1 || D < 4 || D > 512 || (D & 3) || q_stride < D || k_stride < D ||
        ((q_stride | k_stride | ldv) & 3) || (long)nkv * D > 0x7fffffffL || ldv < nkv * D || nrot < 0 || nrot > D || (nrot & 1) || work < 0 || work > 1 ||
        (work == 1 && (D & 31)) || rows < 1 || (!pos && !pos_dev && (pos0 < 0 || pos0 > 0x7fffffff - T)) ||
        (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)qo | (uintptr_t)ko) & 15) || ((uintptr_t)cache & (work ? 1 : 7))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if ((long)T * nh >= 12288 && ko && !pos) {
        // a prefill-sized batch: the kernels that share a token's cos / sin among its heads are 2 - 3 times faster than a wave per head
        // (32 + 4 heads of 128: equal at 256 tokens, 16.7 against 23.5 us at 512, 58 against 166 us at 4096), and the caller's k buffer is
        // there to pass the normed k on
        NrArgs ak = {k, k_stride, nkv, wk, D, nrot, theta_scale, eps, pos0, nullptr, ko, T, pos_dev};
        launch_nr(ak, 0, st);
        const int M = nkv * D;
        const int rc = work ? camx_i_pf_kv_append(ko, M, v, ldv, M, (uint8_t *)cache, pos0, pos_dev, rows, err, T, st)
                            : camx_i_kv_append16(ko, M, v, ldv, (uint16_t *)cache, M, pos0, pos_dev, rows, err, T, st);
        if (rc) return rc;
        NrArgs aq = {q, q_stride, nh, wq, D, nrot, theta_scale, eps, pos0, nullptr, qo, T, pos_dev};
        launch_nr(aq, 0, st);
        CAMX_LAUNCH_RET();
    }
    NrArgs a = {q, q_stride, nh, wq, D, nrot, theta_scale, eps, pos0, pos, qo, T, pos_dev, k, k_stride, nkv, wk, ko, v, ldv, cache, rows, err};
    const long waves = (long)T * (nh + 2 * nkv);
    if ((waves + 3) / 4 > 0x7fffffffL) return CAMX_EINVAL;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (work) qk_nr_heads<false, true, 2><<<grid, block, 0, st>>>(a); else qk_nr_heads<false, true, 1><<<grid, block, 0, st>>>(a);
    CAMX_LAUNCH_RET();
}
// The dense Q8 line's six segments in one launch (see qk_nr_q8_k): heads of 256 dims. q [T][nh] heads at q_stride floats (the q | gate
// interleave), k and v [T][nkv * 256] at ldk / ldv; qo fp32 [T][nh][256] = H256(rotary(norm(q) * qn)); cache row pos + t = Q8 blocks of
// H256(rotary(norm(k) * kn)) per head | Q8 blocks of H64(v) per 64 values. err bits: 1 a row outside [0, rows) (not written; qo is),
// 2 a refused block (bytes untouched). nrot in {16, 32, 64, 128, 256}.
int camx_qk_nr_q8(const float * q, int q_stride, int nh, const float * k, int ldk, const float * v, int ldv, int nkv, const float * qn, const float * kn,
                  int nrot, float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, float * qo, uint8_t * cache, int rows,
                  int * err, int T, hipStream_t st) {
    if (!q || !k || !v || !qn || !kn || !qo || !cache || !err || T < 0 || nh < 1 || nkv < 1 || q_stride < 256 || (q_stride & 3) || ldk < nkv * 256 || ldv < nkv * 256 ||
        ((ldk | ldv) & 3) || rows < 1 || (!pos && !pos_dev && (pos0 < 0 || pos0 > 0x7fffffff - T)) ||
        (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)qn | (uintptr_t)kn | (uintptr_t)qo) & 15) || ((uintptr_t)cache & 1)) return CAMX_EINVAL;
    if (nrot != 16 && nrot != 32 && nrot != 64 && nrot != 128 && nrot != 256) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    NrQ8Args a = {q, q_stride, nh, k, ldk, v, ldv, nkv, qn, kn, theta_scale, eps, pos0, pos_dev, pos, qo, cache, rows, err, T};
    const dim3 grid((unsigned)((long)T * ((nh + 2 * nkv + 7) / 8))), block(256);
    switch (nrot) {
    case 16: qk_nr_q8_k<1><<<grid, block, 0, st>>>(a); break;
    case 32: qk_nr_q8_k<2><<<grid, block, 0, st>>>(a); break;
    case 64: qk_nr_q8_k<4><<<grid, block, 0, st>>>(a); break;
    case 128: qk_nr_q8_k<8><<<grid, block, 0, st>>>(a); break;
    default: qk_nr_q8_k<16><<<grid, block, 0, st>>>(a); break;
    }
    CAMX_LAUNCH_RET();
}
// The OP_OWN_ATTS prologue with the tape's device-resident position (kernels/k3_own_atts.h:183-274; Seg.asum = pos int32 [1]): token t at
// pos[0] + t, checked on the device against the cache's `rows` (err bit 1, the row is not written; q16 is). q8 selects the row format.
int camx_op_own_qk_rope(const float * qkv, int ldq, int nh, int nkv, const float * par, const int32_t * pos, uint16_t * q16, void * cache, int rows,
                        int * err, int n, int yarn, int q8, hipStream_t st) {
    if (!pos) return CAMX_EINVAL;
    RopeArgs a = {qkv, ldq, nh, nkv, par, 0, nullptr, q16, cache, err, nullptr, 0, 0, 0, n, rows, pos};
    return rope_launch(a, yarn, q8 != 0, st);
}
// the per-pair frequencies the rotary kernels use: out[j] = (float)pow((double)theta_scale, j), j < n
int camx_rope_freqs(float theta_scale, int n, float * out, hipStream_t st) {
    if (!out || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    rope_freqs_k<<<dim3((n + 63) / 64), dim3(64), 0, st>>>(theta_scale, n, out);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
