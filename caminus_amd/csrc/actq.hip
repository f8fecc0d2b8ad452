// Fused activation fake-quant for gfx950, forward and backward: per row of K values (K % 128 == 0, K <= 8192) a 128-point
// Hadamard rotation per chunk in bf16 steps, one int4-style scale per row, codes packed two per byte. Replaces actq_fwd_{f32,bf16},
// actq_fwd_codes_{f32,bf16}, actq_bwd_{f32,bf16}, silu_mul_actq_{fwd,bwd} and block_entry_{fwd,bwd} (kernels/actq.hip:40-53,
// 96-218, 247-333).
//
// Rows of at most 2048 values with 16-byte aligned operands, forward and backward, plain and SiLU-fused: one wave per row
// (actq_fwd_wave_k, actq_bwd_wave_k; 30 vector instructions per value against 44 forward, 63 against 78 backward), the fused
// forms with the gates' tables in LDS. Everything else (longer rows, the RMSNorm-fused block entry, unaligned operands):
// One 256-thread workgroup per row. A half-wave (32 lanes) transforms one 128-chunk: lane l holds elements 4l .. 4l + 3,
// butterfly stages 1-2 in registers, 4 .. 64 across lanes; half-wave h takes chunks h, h + 8, ... (the reference's wave h of
// 32), NR = ceil(K / 1024) rounds of them stay in registers across the row-wide reductions. Kernels are instantiated per
// NR, so a row of 2048 values runs two rounds and not the eight the limit allows.
//
// Sums of the backward pass (dL/ds, the tie count, the RMSNorm dot) follow one fixed tree: a lane adds its terms in chunk
// order with fmaf, the 32 lanes of a half-wave combine by xor 16, 8, 4, 2, 1, the eight half-wave sums are added in order.
#include "common.cuh"
#include <mutex>
#include <type_traits>

#define HSCALE 0.08837890625f      // bf16(1 / sqrt(128))

#define CAMX_EACH4(OP) OP(x) OP(y) OP(z) OP(w)

// fp32 -> bf16 -> fp32. _any: a NaN stays a NaN but its sign and payload are the hardware's (for values that only feed further
// arithmetic, where nothing but NaN-ness survives); _canon: a NaN becomes 0x7fc00000, as the stored bf16 tensors have it
CAMX_DEV f32x4 rbf4_any(f32x4 v) {
    const uint32_t a = hw_pk_bf16(v.x, v.y), b = hw_pk_bf16(v.z, v.w);
    f32x4 r;
    r.x = __builtin_bit_cast(float, a << 16); r.y = __builtin_bit_cast(float, a & 0xffff0000u);
    r.z = __builtin_bit_cast(float, b << 16); r.w = __builtin_bit_cast(float, b & 0xffff0000u);
    return r;
}
CAMX_DEV f32x4 rbf4_canon(f32x4 v) { return unpack_bf16x4(pack_f2bf_x4(v)); }
CAMX_DEV f32x4 scaled4(f32x4 v) { v.x *= HSCALE; v.y *= HSCALE; v.z *= HSCALE; v.w *= HSCALE; return v; }

// A source gives four values at element k of a row (operator()), or, for the wave-per-row kernel, eight: fetch() issues the
// loads (NW 128-bit words), value8() turns them into floats later, so that the next row's loads fly during this row's arithmetic.
CAMX_DEV void unpack_bf16x8(u32x4 w, f32x4 & a, f32x4 & b) { a = unpack_bf16x4((u32x2){w.x, w.y}); b = unpack_bf16x4((u32x2){w.z, w.w}); }
struct PlainF32 {
    static constexpr bool bf16_valued = false, lds_tables = false; static constexpr int NW = 2;
    CAMX_DEV void set_small(const uint16_t *) {}
    const float * x; int K;
    CAMX_DEV f32x4 operator()(int row, int k) const { return *(const f32x4 *)(x + (size_t)row * K + k); }
    CAMX_DEV f32x4 operator()(int row, int k, u32x2 &) const { return (*this)(row, k); }
    CAMX_DEV void fetch(int row, int k, u32x4 (&w)[NW]) const { const u32x4 * p = (const u32x4 *)(x + (size_t)row * K + k); w[0] = p[0]; w[1] = p[1]; }
    CAMX_DEV void value8(const u32x4 (&w)[NW], f32x4 & a, f32x4 & b, u32x4 &) const { a = __builtin_bit_cast(f32x4, w[0]); b = __builtin_bit_cast(f32x4, w[1]); }
};
struct PlainBF16 {
    static constexpr bool bf16_valued = true, lds_tables = false; static constexpr int NW = 1;
    CAMX_DEV void set_small(const uint16_t *) {}
    const uint16_t * x; int K;
    CAMX_DEV f32x4 operator()(int row, int k) const { return unpack_bf16x4(*(const u32x2 *)(x + (size_t)row * K + k)); }
    CAMX_DEV f32x4 operator()(int row, int k, u32x2 &) const { return (*this)(row, k); }
    CAMX_DEV void fetch(int row, int k, u32x4 (&w)[NW]) const { w[0] = *(const u32x4 *)(x + (size_t)row * K + k); }
    CAMX_DEV void value8(const u32x4 (&w)[NW], f32x4 & a, f32x4 & b, u32x4 &) const { unpack_bf16x8(w[0], a, b); }
};
// the bf16 words {t[g0], t[g1]} and {t[g2], t[g3]} of four packed bf16 gates: from the small table in LDS when there is one and it
// holds all four, else from the full table in device memory
CAMX_DEV u32x2 silu_lookup4(u32x2 gw, const uint16_t * small, const uint16_t * lut) {
    u32x2 r;
    bool outside = true;
    if (small) {                                                           // (the index of a gate outside the table is a valid entry too)
        outside = false;
        const uint32_t i01 = small_index2(gw.x, outside), i23 = small_index2(gw.y, outside);
        r.x = (uint32_t)small[i01 & 0xffffu] | ((uint32_t)small[i01 >> 16] << 16);
        r.y = (uint32_t)small[i23 & 0xffffu] | ((uint32_t)small[i23 >> 16] << 16);
    }
    if (outside) {
        r.x = (uint32_t)lut[gw.x & 0xffffu] | ((uint32_t)lut[gw.x >> 16] << 16);
        r.y = (uint32_t)lut[gw.y & 0xffffu] | ((uint32_t)lut[gw.y >> 16] << 16);
    }
    return r;
}
struct SiluMulSrc {
    static constexpr bool bf16_valued = true;      // the activation is rounded to bf16 as it is formed
    static constexpr bool lds_tables = true;       // the wave-per-row kernels hold the small tables in LDS
    CAMX_DEV void set_small(const uint16_t * p) { small = p; }
    const uint16_t * gu; int ld, F;
    const uint16_t * lut;                          // bf16(silu g) for every bf16 g (the table silu_mul_bf16 uses: the same activation bits)
    const uint16_t * small;                        // its small form in LDS, or null
    CAMX_DEV f32x4 operator()(int row, int k, u32x2 & keep) const {          // keep: the four bf16(silu g), for the backward's sink
        const uint16_t * r = gu + (size_t)row * ld;
        const u32x2 gw = *(const u32x2 *)(r + k);
        const f32x4 u = unpack_bf16x4(*(const u32x2 *)(r + F + k));
        keep = silu_lookup4(gw, small, lut);
        const f32x4 sl = unpack_bf16x4(keep);
        return rbf4_any((f32x4){sl.x * u.x, sl.y * u.y, sl.z * u.z, sl.w * u.w});      // (feeds the rotation: of a NaN only its NaN-ness survives)
    }
    CAMX_DEV f32x4 operator()(int row, int k) const { u32x2 keep; return (*this)(row, k, keep); }
    static constexpr int NW = 2;                   // the wave-per-row form: eight gates, eight multipliers
    CAMX_DEV void fetch(int row, int k, u32x4 (&w)[NW]) const { const uint16_t * r = gu + (size_t)row * ld + k; w[0] = *(const u32x4 *)r; w[1] = *(const u32x4 *)(r + F); }
    CAMX_DEV void value8(const u32x4 (&w)[NW], f32x4 & a, f32x4 & b, u32x4 & keep) const {
        const u32x2 k0 = silu_lookup4((u32x2){w[0].x, w[0].y}, small, lut), k1 = silu_lookup4((u32x2){w[0].z, w[0].w}, small, lut);
        keep = (u32x4){k0.x, k0.y, k1.x, k1.y};
        f32x4 sa, sb, ua, ub;
        unpack_bf16x8(keep, sa, sb); unpack_bf16x8(w[1], ua, ub);
        a = rbf4_any((f32x4){sa.x * ua.x, sa.y * ua.y, sa.z * ua.z, sa.w * ua.w});
        b = rbf4_any((f32x4){sb.x * ub.x, sb.y * ub.y, sb.z * ub.z, sb.w * ub.w});
    }
};
struct RmsSrc {
    static constexpr bool bf16_valued = false;
    const float * x; const float * w; float rstd; int d;
    CAMX_DEV f32x4 operator()(int row, int k) const {
        const f32x4 xv = *(const f32x4 *)(x + (size_t)row * d + k), wv = *(const f32x4 *)(w + k);
        f32x4 a; a.x = xv.x * rstd * wv.x; a.y = xv.y * rstd * wv.y; a.z = xv.z * rstd * wv.z; a.w = xv.w * rstd * wv.w;
        return a;
    }
    CAMX_DEV f32x4 operator()(int row, int k, u32x2 &) const { return (*this)(row, k); }
};
// The same source for a row that one wave holds in registers (rows of at most 256 NR values): round c of the lane is elements
// 256 c + 4 slot .. + 3, the elements the lane holds in the row's sum of squares and in the projections, so x and the norm
// weights are read once.
template <int NR>
struct RmsRegSrc {
    static constexpr bool bf16_valued = false;
    static constexpr bool by_round = true;
    f32x4 xk[NR], wk[NR]; float rstd;
    CAMX_DEV f32x4 at(int c) const {
        f32x4 a; a.x = xk[c].x * rstd * wk[c].x; a.y = xk[c].y * rstd * wk[c].y; a.z = xk[c].z * rstd * wk[c].z; a.w = xk[c].w * rstd * wk[c].w;
        return a;
    }
    CAMX_DEV f32x4 operator()(int, int k, u32x2 &) const { return at(k >> 8); }
};
template <typename S, typename = void> struct SrcByRound : std::false_type {};
template <typename S> struct SrcByRound<S, std::void_t<decltype(S::by_round)>> : std::true_type {};

// u = bf16(H128 . bf16(source)) for the NR rounds of this half-wave; returns the lane's max |u| over its active chunks
// NHW: the half-waves that share a row (8: a 256-thread workgroup; 2: one wave); half-wave hw takes chunks hw, hw + NHW, ...
template <int NR, typename Src, int NHW = 8>
CAMX_DEV float actq_rotate(Src src, int row, int l, int hw, int nch, f32x4 (&u)[NR], u32x2 * keep = nullptr) {
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int ch = hw + NHW * c;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        u32x2 kp = {0u, 0u};
        if (ch < nch) {
            if constexpr (SrcByRound<Src>::value) { static_assert(NHW == 2, "a wave per row"); v = src.at(c); }
            else v = src(row, ch * 128 + 4 * l, kp);
        }
        if (keep) keep[c] = kp;
        u[c] = v;
    }
    float amax = 0.0f;
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const f32x4 in = Src::bf16_valued ? u[c] : rbf4_any(u[c]);                // autocast's bf16 input
        const f32x4 v = rbf4_any(scaled4(hadamard128_l4(in, l, false)));
        u[c] = v;
        if (hw + NHW * c < nch) amax = fmaxf(amax, absmax4(v));
    }
    return amax;
}

// rintf(u / s) for a lane's four values. p = u * rcp(s) is within 8e-5 of the exact quotient while |p| < 256 (rcp: 1 ulp; one
// more rounding), the IEEE quotient within 1.6e-5 of it, and half-integers are floats: when p is farther than 3e-4 from every
// half-integer, rintf of the two agree. Other lanes (about one value in 1600, and infinities / NaN) divide.
CAMX_DEV f32x4 rint_div4(f32x4 u, float s, float s_rcp) {
    f32x4 p = {u.x * s_rcp, u.y * s_rcp, u.z * s_rcp, u.w * s_rcp};
    f32x4 r = {rintf(p.x), rintf(p.y), rintf(p.z), rintf(p.w)};
    bool safe = true;
#define S_(e) safe &= (fabsf(p.e - r.e) <= 0.4997f) & (fabsf(p.e) < 256.0f);
    CAMX_EACH4(S_)
#undef S_
    if (!safe) { r.x = rintf(u.x / s); r.y = rintf(u.y / s); r.z = rintf(u.z / s); r.w = rintf(u.w / s); }
    return r;
}

// row-wide max (order-free); lds: 4 floats
template <int NHW = 8>
CAMX_DEV float row_max(float amax, float * lds) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    if (NHW == 2) return amax;                           // the row is this wave's
    __syncthreads();
    if ((tid & 63) == 0) lds[tid >> 6] = amax;
    __syncthreads();
    return fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
}

template <int NR, typename Src, int NHW = 8>
CAMX_DEV void actq_fwd_row(Src src, int row, uint16_t * __restrict__ y, float * __restrict__ s_out, int K, float clip, int qmax,
                           uint16_t * __restrict__ codes, float * lds) {
    const int tid = threadIdx.x, l = slot_of(tid) & 31, hw = tid >> 5, nch = K / 128;
    f32x4 u[NR];
    const float amax = row_max<NHW>(actq_rotate<NR, Src, NHW>(src, row, l, hw, nch, u), lds);
    const float s = fmaxf(amax * clip / (float)qmax, 1e-8f), s_rcp = __builtin_amdgcn_rcpf(s);
    if (tid == 0 && s_out) s_out[row] = s;
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int ch = hw + NHW * c;
        if (ch < nch) {
            f32x4 q;
            f32x4 r = rint_div4(u[c], s, s_rcp);
#define Q_(e) q.e = fminf(fmaxf(r.e, lo), hi);
            CAMX_EACH4(Q_)
#undef Q_
            if (y) { f32x4 d; d.x = q.x * s; d.y = q.y * s; d.z = q.z * s; d.w = q.w * s; *(u32x2 *)(y + (size_t)row * K + ch * 128 + 4 * l) = pack_f2bf_x4(d); }
            if (codes) {
                const uint32_t pk = ((uint32_t)(int)q.x & 0xfu) | (((uint32_t)(int)q.y & 0xfu) << 4) | (((uint32_t)(int)q.z & 0xfu) << 8) | (((uint32_t)(int)q.w & 0xfu) << 12);
                codes[(size_t)row * (K / 4) + ch * 32 + l] = (uint16_t)pk;
            }
        }
    }
}

template <int NR, typename Src>
__global__ void __launch_bounds__(256) actq_fwd_k(Src src, uint16_t * y, float * s, uint16_t * codes, int K, float clip, int qmax) {
    __shared__ float lds[4];
    actq_fwd_row<NR>(src, blockIdx.x, y, s, K, clip, qmax, codes, lds);
}

// ---- rows of at most 2048 values: one wave per row, no LDS, no barrier ------------------------------------------------------
// Lane (c = lane >> 2, q = lane & 3) holds 32 values of chunk c: element 32 j + 8 q + k of the chunk is u[j][k]. Butterfly
// stages 1, 2, 4 pair registers k, stages 8 and 16 pair lanes q ^ 1 and q ^ 2, stages 32 and 64 pair registers j: the same
// pairs in the same order as above, five of the seven stages without a lane exchange.
CAMX_DEV void bfly(float & a, float & b) { const float s = a + b, d = a - b; a = s; b = d; }

template <int CTRL>
CAMX_DEV void lane_stage_w(float (&u)[4][8], uint32_t sign) {      // (own + partner) in the lower lane, (partner - own) in the upper one
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float own = u[j][k];
            const float p = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, own), CTRL, 0xf, 0xf, true));
            u[j][k] = p + __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, own) ^ sign);
        }
}
CAMX_DEV void hadamard128_w32(float (&u)[4][8], int q) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int k = 0; k < 8; k += 2) bfly(u[j][k], u[j][k + 1]);
#pragma unroll
        for (int k = 0; k < 8; k += 4) { bfly(u[j][k], u[j][k + 2]); bfly(u[j][k + 1], u[j][k + 3]); }
#pragma unroll
        for (int k = 0; k < 4; k++) bfly(u[j][k], u[j][k + 4]);
    }
    lane_stage_w<0xB1>(u, (q & 1) ? 0x80000000u : 0u);
    lane_stage_w<0x4E>(u, (q & 2) ? 0x80000000u : 0u);
#pragma unroll
    for (int k = 0; k < 8; k++) { bfly(u[0][k], u[1][k]); bfly(u[2][k], u[3][k]); }
#pragma unroll
    for (int k = 0; k < 8; k++) { bfly(u[0][k], u[2][k]); bfly(u[1][k], u[3][k]); }
}
CAMX_DEV float wave_max64(float v) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}
// u = bf16(H128 . bf16(source)) of the lane's 32 values from the fetched words; returns the row's max |u|
template <typename Src>
CAMX_DEV float actq_rotate_w(const Src & src, const u32x4 (&raw)[4][Src::NW], int q, float (&u)[4][8], u32x4 (&keep)[4]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f32x4 a, b;
        src.value8(raw[j], a, b, keep[j]);
        if (!Src::bf16_valued) { a = rbf4_any(a); b = rbf4_any(b); }              // autocast's bf16 input
        u[j][0] = a.x; u[j][1] = a.y; u[j][2] = a.z; u[j][3] = a.w; u[j][4] = b.x; u[j][5] = b.y; u[j][6] = b.z; u[j][7] = b.w;
    }
    hadamard128_w32(u, q);
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int k = 0; k < 8; k += 4) {
            const f32x4 v = rbf4_any(scaled4((f32x4){u[j][k], u[j][k + 1], u[j][k + 2], u[j][k + 3]}));
            u[j][k] = v.x; u[j][k + 1] = v.y; u[j][k + 2] = v.z; u[j][k + 3] = v.w;
            amax = fmaxf(amax, absmax4(v));                                        // (an absent chunk holds zeros)
        }
    return wave_max64(amax);
}
template <typename Src>
CAMX_DEV void fetch_row_w(const Src & src, int row, int c, int q, bool on, u32x4 (&raw)[4][Src::NW]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int w = 0; w < Src::NW; w++) raw[j][w] = (u32x4){0u, 0u, 0u, 0u};
        if (on) src.fetch(row, c * 128 + 32 * j + 8 * q, raw[j]);
    }
}

// a table into LDS, 16 bytes per lane straight from device memory
CAMX_DEV void lds_table_copy(const void * src, void * dst, int bytes) {          // bytes % 1024 == 0; all four waves
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int j = wave; j < bytes / 1024; j += 4)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)((const uint8_t *)src + 1024 * j + 16 * lane),
                                         (__attribute__((address_space(3))) void *)((uint8_t *)dst + 1024 * j), 16, 0, 0);
}
// One row per wave, four rows per workgroup. The kernel's time at 8192 rows is its arithmetic plus the launch's ramp, the first
// loads and the last stores, whatever the number of waves in flight (3 to 8 per SIMD measured alike); a wave that walks several
// rows with the next row's loads in flight measured 5 to 15 % slower.
template <typename Src>
__global__ void __launch_bounds__(256) actq_fwd_wave_k(Src src, uint16_t * __restrict__ y, float * __restrict__ s_out, uint16_t * __restrict__ codes,
                                                       int K, float clip, int qmax, int M, const uint16_t * small_g = nullptr) {
    const int lane = threadIdx.x & 63, nch = K / 128, c = lane >> 2, q = lane & 3;
    const bool on = c < nch;
    const int row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (!Src::lds_tables && row >= M) return;
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
    u32x4 raw[4][Src::NW];
    fetch_row_w(src, min(row, M - 1), c, q, on, raw);
    if (Src::lds_tables) {                               // the gates' table, shared by the workgroup's four rows
        __shared__ __attribute__((aligned(16))) uint16_t small[SWS_TAB];
        lds_table_copy(small_g, small, 2 * SWS_TAB);
        __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0): this wave's part of the table (and its row)
        __syncthreads();
        src.set_small(small);
        if (row >= M) return;
    }
    float u[4][8];
    u32x4 keep[4];                                       // (only the backward uses it)
    const float amax = actq_rotate_w(src, raw, q, u, keep);
    const float s = fmaxf(amax * clip / (float)qmax, 1e-8f), s_rcp = __builtin_amdgcn_rcpf(s);
    if (lane == 0 && s_out) s_out[row] = s;
    if (!on) return;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f32x4 qa = rint_div4((f32x4){u[j][0], u[j][1], u[j][2], u[j][3]}, s, s_rcp), qb = rint_div4((f32x4){u[j][4], u[j][5], u[j][6], u[j][7]}, s, s_rcp);
#define Q_(e) qa.e = fminf(fmaxf(qa.e, lo), hi); qb.e = fminf(fmaxf(qb.e, lo), hi);
        CAMX_EACH4(Q_)
#undef Q_
        const size_t e0 = (size_t)row * K + c * 128 + 32 * j + 8 * q;
        if (y) {
            const u32x2 pa = pack_f2bf_x4((f32x4){qa.x * s, qa.y * s, qa.z * s, qa.w * s}), pb = pack_f2bf_x4((f32x4){qb.x * s, qb.y * s, qb.z * s, qb.w * s});
            *(u32x4 *)(y + e0) = (u32x4){pa.x, pa.y, pb.x, pb.y};
        }
        if (codes) {
#define N_(v, sh) (((uint32_t)(int)(v) & 0xfu) << (sh))
            const uint32_t pk = N_(qa.x, 0) | N_(qa.y, 4) | N_(qa.z, 8) | N_(qa.w, 12) | N_(qb.x, 16) | N_(qb.y, 20) | N_(qb.z, 24) | N_(qb.w, 28);
#undef N_
            *(uint32_t *)(codes + (e0 >> 2)) = pk;
        }
    }
}

// ---- backward ----------------------------------------------------------------------------------------------------------------
// sum over the 32 lanes of a half-wave by xor 16, 8, 4, 2, 1 (slot space), then the eight half-wave sums in order
CAMX_DEV float half32_sum(float v) {
    v += lane_xor16(v); v += lane_xor8(v); v += lane_xor4(v); v += lane_xor2(v); v += lane_xor1(v);
    return v;
}
CAMX_DEV void block8_sum2(float & a, float & b, float * lds16) {
    const int tid = threadIdx.x;
    a = half32_sum(a); b = half32_sum(b);
    __syncthreads();
    if ((tid & 31) == 0) { lds16[tid >> 5] = a; lds16[8 + (tid >> 5)] = b; }
    __syncthreads();
    a = lds16[0]; b = lds16[8];
#pragma unroll
    for (int w = 1; w < 8; w++) { a += lds16[w]; b += lds16[8 + w]; }
}

// u / s for a row's values, s the row's scale: the IEEE quotient by the compiler's own expansion (reciprocal, one Newton step,
// the product and two corrections, each an fma) without its scaling and fix-up steps, which only act when an exponent is
// extreme. Taken when s and max |u| / s lie in [2^-60, 2^60] and the lane's four quotients are at least 2^-60 in magnitude:
// every intermediate is then a normal number and both forms run the same arithmetic (an exhaustive-neighbourhood check on a CPU
// over 10^8 (u, s) pairs, with every reciprocal within an ulp, found no difference). Other lanes divide.
struct RowDiv {
    float s, r1; bool row_ok;
    CAMX_DEV RowDiv(float s_, float amax) : s(s_) {
        const float r0 = __builtin_amdgcn_rcpf(s_);
        r1 = __builtin_fmaf(__builtin_fmaf(-s_, r0, 1.0f), r0, r0);
        row_ok = s_ >= 0x1p-60f && s_ <= 0x1p60f && amax * r1 <= 0x1p60f;
    }
    CAMX_DEV f32x4 div4(f32x4 u, bool needed = true) const {       // needed: false in a lane whose values are padding
        f32x4 t, t0 = {u.x * r1, u.y * r1, u.z * r1, u.w * r1};
#define T_(e) { const float rem = __builtin_fmaf(-s, t0.e, u.e), t1 = __builtin_fmaf(rem, r1, t0.e); t.e = __builtin_fmaf(__builtin_fmaf(-s, t1, u.e), r1, t1); }
        CAMX_EACH4(T_)
#undef T_
        const float least = fminf(fminf(fabsf(t0.x), fabsf(t0.y)), fminf(fabsf(t0.z), fabsf(t0.w)));     // (a NaN quotient is a NaN either way)
        if (needed && !(row_ok && least >= 0x1p-60f)) { t.x = u.x / s; t.y = u.y / s; t.z = u.z / s; t.w = u.w / s; }
        return t;
    }
};

struct SinkF32 {
    float * dx; int K;
    CAMX_DEV void operator()(int row, int k, f32x4 v, u32x2) const { *(f32x4 *)(dx + (size_t)row * K + k) = v; }
    CAMX_DEV void st8(int row, int k, f32x4 a, f32x4 b, u32x4) const { f32x4 * p = (f32x4 *)(dx + (size_t)row * K + k); p[0] = a; p[1] = b; }
    CAMX_DEV void set_small(const float *) {}
};
struct SinkBF16 {
    uint16_t * dx; int K;
    CAMX_DEV void operator()(int row, int k, f32x4 v, u32x2) const { *(u32x2 *)(dx + (size_t)row * K + k) = pack_f2bf_x4(v); }
    CAMX_DEV void st8(int row, int k, f32x4 a, f32x4 b, u32x4) const {
        const u32x2 pa = pack_f2bf_x4(a), pb = pack_f2bf_x4(b);
        *(u32x4 *)(dx + (size_t)row * K + k) = (u32x4){pa.x, pa.y, pb.x, pb.y};
    }
    CAMX_DEV void set_small(const float *) {}
};
struct SinkLds { float * buf; CAMX_DEV void operator()(int, int k, f32x4 v, u32x2) const { *(f32x4 *)(buf + k) = v; } };
// dact back through act = bf16(bf16(silu g) * u): each product rounded to bf16, then silu's derivative
// ds * sig * fma(g, 1 - sig, 1), into dgu = [dg | du] rows of 2F. g is a bf16 value, so sig = 1 / (1 + expf(-g))
// is read from a table of all 65536 of them (filled on first use from the correctly rounded expf): one 4-byte load in place of an
// exponential and a division per value; the wave-per-row kernel holds the table's small form in LDS. (A table in device memory
// that also holds the fma doubles the entry, and the values in use no longer stay in the first-level cache: 15 % slower than
// no table at all.)
__device__ __attribute__((aligned(16))) float g_dsilu_lut[65536];
__device__ __attribute__((aligned(16))) float g_dsilu_small[SWS_TAB];            // the small form, for LDS
__global__ void __launch_bounds__(256) dsilu_lut_fill() {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    const float g = bf2f((uint16_t)i), ex = (float)exp(-(double)g), sig = 1.0f / (1.0f + ex);
    g_dsilu_lut[i] = sig;
}
__global__ void __launch_bounds__(256) dsilu_small_fill() {              // after dsilu_lut_fill, on the same stream
    const uint32_t e = blockIdx.x * 256 + threadIdx.x;
    if (e >= SWS_TAB) return;
    const uint32_t sign = e >> 12, i = e & SWS_SPAN;
    g_dsilu_small[e] = g_dsilu_lut[i == SWS_SPAN ? sign << 15 : (sign << 15) | (SWS_A0 + i)];
}
struct SinkSiluMul {
    const uint16_t * gu; int ld, F; uint16_t * dgu; const float * dlut;
    const float * dsmall;                          // the small sigmoid table in LDS, or null
    CAMX_DEV void set_small(const float * p) { dsmall = p; }
    CAMX_DEV void operator()(int row, int k, f32x4 dact, u32x2 keep) const {      // keep: the source's four bf16(silu g)
        const uint16_t * r = gu + (size_t)row * ld;
        u32x2 dgp, dup;
        grads4(*(const u32x2 *)(r + k), *(const u32x2 *)(r + F + k), keep, dact, dgp, dup);
        uint16_t * o = dgu + (size_t)row * (2 * F);
        *(u32x2 *)(o + k) = dgp;
        *(u32x2 *)(o + F + k) = dup;
    }
    // four values' dg and du from their gates, multipliers, bf16(silu g) and dact
    CAMX_DEV void grads4(u32x2 gw, u32x2 uw, u32x2 keep, f32x4 dact, u32x2 & dgp, u32x2 & dup) const {
        const f32x4 g = unpack_bf16x4(gw), u = unpack_bf16x4(uw), sl4 = unpack_bf16x4(keep);
        bool outside = true;
        f32x4 sig;
        if (dsmall) {
            outside = false;
            const uint32_t i01 = small_index2(gw.x, outside), i23 = small_index2(gw.y, outside);
            sig = (f32x4){dsmall[i01 & 0xffffu], dsmall[i01 >> 16], dsmall[i23 & 0xffffu], dsmall[i23 >> 16]};
        }
        if (outside) sig = (f32x4){dlut[gw.x & 0xffffu], dlut[gw.x >> 16], dlut[gw.y & 0xffffu], dlut[gw.y >> 16]};
        const f32x4 ds = rbf4_any((f32x4){dact.x * u.x, dact.y * u.y, dact.z * u.z, dact.w * u.w});       // (a NaN's bits are settled by the store's rounding)
        f32x4 dg, du;
#define S_(e) { du.e = dact.e * sl4.e; dg.e = ds.e * sig.e * __builtin_fmaf(g.e, 1.0f - sig.e, 1.0f); }
        CAMX_EACH4(S_)
#undef S_
        dgp = pack_f2bf_x4(dg); dup = pack_f2bf_x4(du);
    }
    // (the gates and multipliers are read a second time here: held in registers since the source fetched them they cost 48 more,
    // two waves per SIMD instead of three, and 8192 x 2048 takes 65 us instead of 62)
    CAMX_DEV void st8(int row, int k, f32x4 a, f32x4 b, u32x4 keep) const {
        const uint16_t * r = gu + (size_t)row * ld + k;
        const u32x4 gw = *(const u32x4 *)r, uw = *(const u32x4 *)(r + F);
        u32x2 dg0, du0, dg1, du1;
        grads4((u32x2){gw.x, gw.y}, (u32x2){uw.x, uw.y}, (u32x2){keep.x, keep.y}, a, dg0, du0);
        grads4((u32x2){gw.z, gw.w}, (u32x2){uw.z, uw.w}, (u32x2){keep.z, keep.w}, b, dg1, du1);
        uint16_t * o = dgu + (size_t)row * (2 * F) + k;
        *(u32x4 *)o = (u32x4){dg0.x, dg0.y, dg1.x, dg1.y};
        *(u32x4 *)(o + F) = (u32x4){du0.x, du0.y, du1.x, du1.y};
    }
};

// lds16: 16 floats. sink receives bf16-valued floats: the gradient of the bf16 source, before any widening store.
// NHW = 8: a 256-thread workgroup per row. NHW = 2: one wave per row of at most 1024 values (each half-wave sum of the tree is
// then one chunk's: round c holds chunks 2 c and 2 c + 1); out, when given, receives round c's result in place of the sink.
template <int NR, typename Src, typename Sink, int NHW = 8>
CAMX_DEV void actq_bwd_row(Src src, int row, const uint16_t * __restrict__ g, Sink sink, int K, float clip, int qmax, float * lds16, f32x4 * out = nullptr) {
    const int tid = threadIdx.x, l = slot_of(tid) & 31, hw = tid >> 5, nch = K / 128;
    f32x4 u[NR], gv[NR];
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int ch = hw + NHW * c;
        u32x2 raw = {0u, 0u};
        if (ch < nch) raw = *(const u32x2 *)(g + (size_t)row * K + ch * 128 + 4 * l);
        gv[c] = unpack_bf16x4(raw);
    }
    u32x2 keep[NR];                                      // what the source hands to the sink (the fused SiLU form only)
    const float amax = row_max<NHW>(actq_rotate<NR, Src, NHW>(src, row, l, hw, nch, u, keep), lds16);
    const float s_raw = amax * clip / (float)qmax, s = fmaxf(s_raw, 1e-8f);
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
    // dL/ds = sum g (q - m t) and the number of max-|u| elements; m: the rounded value lies strictly inside (lo, hi). The
    // straight-through part g m is formed here (g is not needed afterwards); the ties are counted from the compares' lane masks
    // on the scalar unit, one counter per half-wave (a count is exact in any order).
    const RowDiv rd(s, amax);
    float dlds = 0.0f, part[NHW == 2 ? NR : 1];           // NHW == 2: a sum per round (a reference lane's terms are one chunk's)
    int ties_lo = 0, ties_hi = 0;
    uint32_t tied = 0;                                   // bit c: some lane of this wave holds a max-|u| element in round c
#pragma unroll
    for (int c = 0; c < NR; c++) {
        if (NHW == 2) dlds = 0.0f;
        if (hw + NHW * c < nch) {
            const f32x4 t4 = rd.div4(u[c]);
            uint64_t any = 0;
#define D_(e) { const float t = t4.e, r = rintf(t), q = fminf(fmaxf(r, lo), hi); const bool m = r > lo && r < hi; \
                dlds = __builtin_fmaf(gv[c].e, m ? q - t : q, dlds); gv[c].e = gv[c].e * (m ? 1.0f : 0.0f); \
                const uint64_t tie = __builtin_amdgcn_ballot_w64(fabsf(u[c].e) == amax); any |= tie; \
                ties_lo += __builtin_popcount((uint32_t)tie); ties_hi += __builtin_popcount((uint32_t)(tie >> 32)); }
            CAMX_EACH4(D_)
#undef D_
            if (any) tied |= 1u << c;
        }
        if (NHW == 2) part[NHW == 2 ? c : 0] = dlds;
    }
    float ties;
    if (NHW == 2) {                                      // the eight chunk sums in order (absent chunks add +0, as idle half-waves do)
        ties = lane_read((float)(ties_lo + ties_hi), 0);          // lane 0's count: its half-wave is in every round that any lane is in (the counters of a lane that sits out a round miss that round)
#pragma unroll
        for (int c = 0; c < NR; c++) {
            const float hs = half32_sum(part[NHW == 2 ? c : 0]);
            const float even = lane_read(hs, 0), odd = lane_read(hs, 32);
            dlds = c == 0 ? even : dlds + even;
            dlds += odd;
        }
        if (2 * NR < 8) dlds += 0.0f;
    } else {
        ties = (tid & 31) == 0 ? (float)((tid & 32) ? ties_hi : ties_lo) : 0.0f;
        block8_sum2(dlds, ties, lds16);
    }
    const float coef = s_raw >= 1e-8f ? dlds * clip / (float)qmax / ties : 0.0f;
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int ch = hw + NHW * c;
        if (out) out[c] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        if (ch < nch) {
            f32x4 d = gv[c];
            if (tied & (1u << c)) {                      // wave-uniform: a row has few such elements, most rounds skip this
#define V_(e) if (fabsf(u[c].e) == amax && u[c].e != 0.0f) d.e += u[c].e > 0.0f ? coef : -coef;
                CAMX_EACH4(V_)
#undef V_
            }
            const f32x4 r = rbf4_canon(scaled4(hadamard128_l4(rbf4_any(d), l, false)));      // rbf4_any: the gradient of the bf16 tensor u
            if (out) out[c] = r; else sink(row, ch * 128 + 4 * l, r, keep[c]);
        }
    }
}

template <int NR, typename Src, typename Sink>
__global__ void __launch_bounds__(256) actq_bwd_k(Src src, const uint16_t * g, Sink sink, int K, float clip, int qmax) {
    __shared__ float lds[16];
    actq_bwd_row<NR>(src, blockIdx.x, g, sink, K, clip, qmax, lds);
}

// ---- backward of rows of at most 2048 values: one wave per row, in the layout of actq_fwd_wave_k ------------------------------------
// The sum of dL/ds keeps the tree of the workgroup form. There, the lane of half-wave h with index l adds the terms of elements
// 4 l .. 4 l + 3 of chunk h, then of chunk h + 8, in order; here those eight terms sit in two lanes (c = h and c = h + 8, 32 lanes
// apart) as registers 4 kk .. 4 kk + 3 of group j, with l = 8 j + 2 q + kk. Every lane runs the four-term chain from zero, the upper
// 32 lanes fetch the lower lanes' results and run theirs again from there. The 32 sums of a half-wave then combine by
// l ^ 16, 8 (registers j), 4, 2 (lanes q), 1 (registers kk), and the eight half-wave sums, held by lanes 32 + 4 h, are added in order.
CAMX_DEV float from_other_half(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * (lane ^ 32), __builtin_bit_cast(int, v)));
}
template <typename Src, typename Sink>
__global__ void __launch_bounds__(256) actq_bwd_wave_k(Src src, const uint16_t * __restrict__ g, Sink sink, int K, float clip, int qmax, int M,
                                                       const uint16_t * small_g = nullptr, const float * dsmall_g = nullptr) {
    const int lane = threadIdx.x & 63, nch = K / 128, c = lane >> 2, q = lane & 3;
    const bool on = c < nch, upper = lane >= 32;
    const int row_raw = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (!Src::lds_tables && row_raw >= M) return;
    const int row = min(row_raw, M - 1);
    u32x4 raw[4][Src::NW], graw[4];
    fetch_row_w(src, row, c, q, on, raw);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        graw[j] = (u32x4){0u, 0u, 0u, 0u};
        if (on) graw[j] = *(const u32x4 *)(g + (size_t)row * K + c * 128 + 32 * j + 8 * q);
    }
    if (Src::lds_tables) {                               // the gates' tables, shared by the workgroup's four rows
        __shared__ __attribute__((aligned(16))) uint16_t small[SWS_TAB];
        __shared__ __attribute__((aligned(16))) float dsmall[SWS_TAB];
        lds_table_copy(small_g, small, 2 * SWS_TAB);
        lds_table_copy(dsmall_g, dsmall, 4 * SWS_TAB);
        __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0): this wave's part of the tables (and its row)
        __syncthreads();
        src.set_small(small); sink.set_small(dsmall);
        if (row_raw >= M) return;
    }
    float u[4][8];
    u32x4 keep[4];
    const float amax = actq_rotate_w(src, raw, q, u, keep);
    const float s_raw = amax * clip / (float)qmax, s = fmaxf(s_raw, 1e-8f);
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
    const RowDiv rd(s, amax);
    const uint64_t on_mask = __builtin_amdgcn_ballot_w64(on);
    float gm[4][8], part[4][2];                          // g m; the reference lanes' sums of dL/ds terms
    int ties_n = 0;
    uint32_t tied = 0;                                   // bit j: group j holds a max-|u| element in some lane
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f32x4 ga, gb;
        unpack_bf16x8(graw[j], ga, gb);
        const float g8[8] = {ga.x, ga.y, ga.z, ga.w, gb.x, gb.y, gb.z, gb.w};
        const f32x4 ta = rd.div4((f32x4){u[j][0], u[j][1], u[j][2], u[j][3]}, on), tb = rd.div4((f32x4){u[j][4], u[j][5], u[j][6], u[j][7]}, on);
        const float t8[8] = {ta.x, ta.y, ta.z, ta.w, tb.x, tb.y, tb.z, tb.w};
        float x8[8];
        uint64_t any = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float t = t8[k], r = rintf(t), qv = fminf(fmaxf(r, lo), hi);
            const bool m = r > lo && r < hi;
            x8[k] = m ? qv - t : qv;
            gm[j][k] = g8[k] * (m ? 1.0f : 0.0f);
            const uint64_t tie = __builtin_amdgcn_ballot_w64(fabsf(u[j][k]) == amax) & on_mask;
            any |= tie;
            ties_n += __builtin_popcountll(tie);
        }
        if (any) tied |= 1u << j;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            float a = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; e++) a = __builtin_fmaf(g8[4 * kk + e], x8[4 * kk + e], a);
            const float below = from_other_half(a, lane);
            float b = below;
#pragma unroll
            for (int e = 0; e < 4; e++) b = __builtin_fmaf(g8[4 * kk + e], x8[4 * kk + e], b);
            part[j][kk] = upper ? (on ? b : below) : a;
        }
    }
    float dlds;
    {
        const float b00 = part[0][0] + part[2][0], b01 = part[0][1] + part[2][1], b10 = part[1][0] + part[3][0], b11 = part[1][1] + part[3][1];   // l ^ 16
        float c0 = b00 + b10, c1 = b01 + b11;                                                                                                      // l ^ 8
        c0 += lane_xor2(c0); c1 += lane_xor2(c1);                                                                                                  // l ^ 4
        c0 += lane_xor1(c0); c1 += lane_xor1(c1);                                                                                                  // l ^ 2
        const float d = c0 + c1;                                                                                                                   // l ^ 1
        dlds = lane_read(d, 32);
#pragma unroll
        for (int h = 1; h < 8; h++) dlds += lane_read(d, 32 + 4 * h);
    }
    const float coef = s_raw >= 1e-8f ? dlds * clip / (float)qmax / (float)ties_n : 0.0f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (tied & (1u << j)) {                          // wave-uniform: a row has few such elements
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (on && fabsf(u[j][k]) == amax && u[j][k] != 0.0f) gm[j][k] += u[j][k] > 0.0f ? coef : -coef;
        }
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int k = 0; k < 8; k += 4) {
            const f32x4 v = rbf4_any((f32x4){gm[j][k], gm[j][k + 1], gm[j][k + 2], gm[j][k + 3]});      // the gradient of the bf16 tensor u
            gm[j][k] = v.x; gm[j][k + 1] = v.y; gm[j][k + 2] = v.z; gm[j][k + 3] = v.w;
        }
    hadamard128_w32(gm, q);
    if (!on) return;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const f32x4 a = rbf4_canon(scaled4((f32x4){gm[j][0], gm[j][1], gm[j][2], gm[j][3]})), b = rbf4_canon(scaled4((f32x4){gm[j][4], gm[j][5], gm[j][6], gm[j][7]}));
        sink.st8(row, c * 128 + 32 * j + 8 * q, a, b, keep[j]);
    }
}

// ---- block entry: h = RMSNorm(x) never materialized ------------------------------------------------------------------------
// row sum under the 256-thread tree, computed by the first wave (elements 256 j + 4 lane + k), result to all threads
template <typename F>
CAMX_DEV float row_tree_sum(F term, int d, float * slot) {
    if (threadIdx.x < 64) {
        const int lane = slot_of(threadIdx.x);
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int base = 0; base < d; base += 256) {
            const int k = base + 4 * lane;
            if (k < d) { const f32x4 a = term(k), b = term.other(k); acc.x = __builtin_fmaf(a.x, b.x, acc.x); acc.y = __builtin_fmaf(a.y, b.y, acc.y);
                         acc.z = __builtin_fmaf(a.z, b.z, acc.z); acc.w = __builtin_fmaf(a.w, b.w, acc.w); }
        }
        const float tot = wave_groups_in_order(group32_sum(acc));
        if (lane == 0) *slot = tot;
    }
    __syncthreads();
    const float r = *slot;
    __syncthreads();
    return r;
}
struct SqTerm { const float * x; CAMX_DEV f32x4 operator()(int k) const { return *(const f32x4 *)(x + k); } CAMX_DEV f32x4 other(int k) const { return *(const f32x4 *)(x + k); } };
struct AbTerm {
    const float * x; const float * w; float rstd; const uint16_t * wab;
    CAMX_DEV f32x4 operator()(int k) const {
        const f32x4 xv = *(const f32x4 *)(x + k), wv = *(const f32x4 *)(w + k);
        f32x4 a; a.x = rbf(xv.x * rstd * wv.x); a.y = rbf(xv.y * rstd * wv.y); a.z = rbf(xv.z * rstd * wv.z); a.w = rbf(xv.w * rstd * wv.w);
        return a;
    }
    CAMX_DEV f32x4 other(int k) const { return unpack_bf16x4(*(const u32x2 *)(wab + k)); }
};

// NHW = 8: a 256-thread workgroup per row (NR rounds of 1024 values); NHW = 2: one wave per row for rows of at most 1024 values (NR
// rounds of 256): a lane then holds 16 values instead of 4, and what every lane computes once per row (the square root, the
// divisions, the reductions' tails, 900 instructions in all) is spread over four times as many values.
// The projections: wave w takes rows w, w + W, ... of wab (W waves per row), up to four of them at a time so that their loads fly together,
// each under the 256-thread tree (a lane holds the logical threads 4 lane .. 4 lane + 3, which add their elements 256 apart in
// order); rows of at most 2048 values keep bf16(h) in registers.
template <int NR, int NHW>
__global__ void __launch_bounds__(32 * NHW) block_entry_fwd_k(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y,
                                                              float * s, uint16_t * codes, uint16_t * ab, float * rstd_out, int d, float clip, int qmax) {
    __shared__ float lds[4];
    __shared__ float slot;
    const int row = blockIdx.x;
    const float * xr = x + (size_t)row * d;
    constexpr int NW = NHW / 2, NA = NR * NHW / 2;       // waves per row; 256-element steps of a row
    constexpr bool KEEP = NA <= 8;
    const int lane = slot_of(threadIdx.x & 63), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    f32x4 hk[KEEP ? NA : 1];
    float rstd;
    if constexpr (NHW == 2) {                            // the row and the norm weights in registers: every HBM byte of x crosses once
        RmsRegSrc<NR> src;
#pragma unroll
        for (int c = 0; c < NR; c++) {
            const int k = 256 * c + 4 * lane;
            src.xk[c] = src.wk[c] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
            if (k < d) { src.xk[c] = __builtin_nontemporal_load((const f32x4 *)(xr + k)); src.wk[c] = *(const f32x4 *)(nw + k); }
        }
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < NR; c++)
            if (256 * c + 4 * lane < d) {
                acc.x = __builtin_fmaf(src.xk[c].x, src.xk[c].x, acc.x); acc.y = __builtin_fmaf(src.xk[c].y, src.xk[c].y, acc.y);
                acc.z = __builtin_fmaf(src.xk[c].z, src.xk[c].z, acc.z); acc.w = __builtin_fmaf(src.xk[c].w, src.xk[c].w, acc.w);
            }
        const float ss = wave_groups_in_order(group32_sum(acc));
        rstd = rsqrt_exact(ss / (float)d + eps);
        src.rstd = rstd;
        if (threadIdx.x == 0 && rstd_out) rstd_out[row] = rstd;
        actq_fwd_row<NR, RmsRegSrc<NR>, NHW>(src, row, y, s, d, clip, qmax, codes, lds);
        if (nab == 0) return;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const f32x4 a = src.at(i % NR);
            hk[KEEP ? i : 0] = 256 * i + 4 * lane < d ? (f32x4){rbf(a.x), rbf(a.y), rbf(a.z), rbf(a.w)} : (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        }
    } else {
        const float ss = row_tree_sum(SqTerm{xr}, d, &slot);
        rstd = rsqrt_exact(ss / (float)d + eps);
        if (threadIdx.x == 0 && rstd_out) rstd_out[row] = rstd;
        actq_fwd_row<NR, RmsSrc, NHW>(RmsSrc{x, nw, rstd, d}, row, y, s, d, clip, qmax, codes, lds);
        if (nab == 0) return;
    }
    const AbTerm term{xr, nw, rstd, wab};
    if (KEEP && NHW != 2) {
#pragma unroll
        for (int i = 0; i < NA; i++) { const int k = 256 * i + 4 * lane; hk[KEEP ? i : 0] = k < d ? term(k) : (f32x4){0.0f, 0.0f, 0.0f, 0.0f}; }
    }
    constexpr int JB = NA <= 4 ? 4 : NA <= 8 ? 2 : 1;   // rows of wab whose loads fly together
    for (int j0 = wave; j0 < nab; j0 += JB * NW) {
        u32x2 wv[JB][NA];
#pragma unroll
        for (int jj = 0; jj < JB; jj++) {
            const int j = j0 + NW * jj;
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int k = 256 * i + 4 * lane;
                wv[jj][i] = (u32x2){0u, 0u};
                if (j < nab && k < d) wv[jj][i] = *(const u32x2 *)(wab + (size_t)j * d + k);
            }
        }
#pragma unroll
        for (int jj = 0; jj < JB; jj++) {
            const int j = j0 + NW * jj;
            if (j >= nab) break;                         // (wave-uniform)
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int k = 256 * i + 4 * lane;
                if (k < d) {
                    const f32x4 a = KEEP ? hk[KEEP ? i : 0] : term(k), b = unpack_bf16x4(wv[jj][i]);
                    acc.x = __builtin_fmaf(a.x, b.x, acc.x); acc.y = __builtin_fmaf(a.y, b.y, acc.y);
                    acc.z = __builtin_fmaf(a.z, b.z, acc.z); acc.w = __builtin_fmaf(a.w, b.w, acc.w);
                }
            }
            const float tot = wave_groups_in_order(group32_sum(acc));
            if ((threadIdx.x & 63) == 0) ab[(size_t)row * nab + j] = f2bf(tot);
        }
    }
}

// dh = actq backward of dy, plus the two projection groups' input gradients (wab rows [0, nab / 2) and [nab / 2, nab), each
// group's sum rounded to bf16); then the RMSNorm backward dx = rstd (dh w - xhat mean(dh w xhat)), xhat = x rstd. d <= 1024.
// One wave per row, NR = ceil(d / 256) rounds: lane (slot la) holds elements 256 c + 4 la .. + 3 of round c through all three steps,
// i.e. the logical threads 4 la .. 4 la + 3 of the 256-thread tree of the dot product (thread t owns elements t, t + 256, ...).
struct SinkNone { CAMX_DEV void operator()(int, int, f32x4, u32x2) const {} };
template <int NR>
__global__ void __launch_bounds__(64) block_entry_bwd_k(const float * x, const float * nw, const float * rstd_in, const uint16_t * wab, int nab,
                                                        const uint16_t * dy, const uint16_t * dab, float * dx, int d, float clip, int qmax) {
    const int row = blockIdx.x, la = slot_of(threadIdx.x);
    const float rstd = rstd_in[row];
    const float * xr = x + (size_t)row * d;
    RmsRegSrc<NR> src;                                   // x and the norm weights once, for the quantizer's source and the RMSNorm backward
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int k = 256 * c + 4 * la;
        src.xk[c] = src.wk[c] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        if (k < d) { src.xk[c] = __builtin_nontemporal_load((const f32x4 *)(xr + k)); src.wk[c] = *(const f32x4 *)(nw + k); }
    }
    src.rstd = rstd;
    f32x4 dh[NR];
    actq_bwd_row<NR, RmsRegSrc<NR>, SinkNone, 2>(src, row, dy, SinkNone{}, d, clip, qmax, nullptr, dh);
    if (nab) {                                           // the projections' part of dh
        const int half = nab / 2;
        float dabs[2][8];                                // the row's dab by group, the same in every lane: scalar registers
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t w = j < half ? (uint32_t)__builtin_amdgcn_readfirstlane((int)dab[(size_t)row * nab + h * half + j]) : 0u;
                dabs[h][j] = __builtin_bit_cast(float, w << 16);
            }
#pragma unroll
        for (int c = 0; c < NR; c++) {
            const int k = 256 * c + 4 * la;
            if (k < d) {
                f32x4 p[2];                              // rows [0, half) of wab add into p[0], [half, nab) into p[1], each in order
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    u32x2 wv[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) { wv[j] = (u32x2){0u, 0u}; if (j < half) wv[j] = *(const u32x2 *)(wab + (size_t)(h * half + j) * d + k); }
                    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        if (j < half) {                  // (uniform)
                            const f32x4 w = unpack_bf16x4(wv[j]);
                            const float cj = dabs[h][j];
                            acc.x = __builtin_fmaf(cj, w.x, acc.x); acc.y = __builtin_fmaf(cj, w.y, acc.y); acc.z = __builtin_fmaf(cj, w.z, acc.z); acc.w = __builtin_fmaf(cj, w.w, acc.w);
                        }
                    }
                    p[h] = acc;
                }
                const f32x4 ra = rbf4_canon(p[0]), rb = rbf4_canon(p[1]);
                f32x4 g = dh[c];
                g.x = (g.x + ra.x) + rb.x; g.y = (g.y + ra.y) + rb.y; g.z = (g.z + ra.z) + rb.z; g.w = (g.w + ra.w) + rb.w;
                dh[c] = g;
            }
        }
    }
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f}, gw[NR], xh[NR];
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int k = 256 * c + 4 * la;
        gw[c] = xh[c] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        if (k < d) {
            const f32x4 w = src.wk[c], xv = src.xk[c];
            gw[c] = (f32x4){dh[c].x * w.x, dh[c].y * w.y, dh[c].z * w.z, dh[c].w * w.w};
            xh[c] = (f32x4){xv.x * rstd, xv.y * rstd, xv.z * rstd, xv.w * rstd};
            acc.x = __builtin_fmaf(gw[c].x, xh[c].x, acc.x); acc.y = __builtin_fmaf(gw[c].y, xh[c].y, acc.y);
            acc.z = __builtin_fmaf(gw[c].z, xh[c].z, acc.z); acc.w = __builtin_fmaf(gw[c].w, xh[c].w, acc.w);
        }
    }
    const float gs = group32_sum(acc);                   // the 32 logical threads of a group, then the eight groups in order
    float dot = lane_read(gs, 0);
#pragma unroll
    for (int q = 1; q < 8; q++) dot += lane_read(gs, 8 * q);
    dot = dot / (float)d;
#pragma unroll
    for (int c = 0; c < NR; c++) {
        const int k = 256 * c + 4 * la;
        if (k < d) {
            f32x4 r;
            r.x = rstd * (gw[c].x - xh[c].x * dot); r.y = rstd * (gw[c].y - xh[c].y * dot);
            r.z = rstd * (gw[c].z - xh[c].z * dot); r.w = rstd * (gw[c].w - xh[c].w * dot);
            *(f32x4 *)(dx + (size_t)row * d + k) = r;
        }
    }
}

__attribute__((visibility("hidden"))) int silu_luts_get(hipStream_t st, const uint16_t ** lut, const uint16_t ** small);       // quant.hip

// the derivative table's device address, filled once per device in stream order before its first reader; callers on any host
// thread go through one lock
static std::mutex g_dlut_mu;
static struct { bool ready; const float * lut; const float * small; } g_dlut_dev[64];
static int dsilu_luts_get(hipStream_t st, const float ** lut, const float ** small) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return CAMX_EINVAL;
    std::lock_guard<std::mutex> lock(g_dlut_mu);
    if (!g_dlut_dev[dev].ready) {
        dsilu_lut_fill<<<dim3(256), dim3(256), 0, st>>>();
        dsilu_small_fill<<<dim3((SWS_TAB + 255) / 256), dim3(256), 0, st>>>();
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
        void * sym = nullptr, * sym_small = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_dsilu_lut)) != hipSuccess || !sym) return CAMX_EINVAL;
        if (hipGetSymbolAddress(&sym_small, HIP_SYMBOL(g_dsilu_small)) != hipSuccess || !sym_small) return CAMX_EINVAL;
        if (hipStreamSynchronize(st) != hipSuccess) return CAMX_EINVAL;     // later calls may come on other streams
        g_dlut_dev[dev].lut = (const float *)sym;
        g_dlut_dev[dev].small = (const float *)sym_small;
        g_dlut_dev[dev].ready = true;
    }
    *lut = g_dlut_dev[dev].lut;
    *small = g_dlut_dev[dev].small;
    return CAMX_OK;
}

__attribute__((visibility("hidden"))) int dsilu_luts_init(hipStream_t st) {       // camx_init's half of this file
    const float * lut = nullptr, * small = nullptr;
    return dsilu_luts_get(st, &lut, &small);
}

// the wave-per-row forward kernel: rows of at most 2048 values, operands aligned for its 16-byte loads and 16- / 4-byte stores
static bool actq_wave_ok(int K, const void * x, const void * y, const void * codes) { return K <= 2048 && !((uintptr_t)x & 15) && !((uintptr_t)y & 15) && !((uintptr_t)codes & 3); }

static int actq_check(int K, int qmax, int M) { return (K < 128 || K % 128 || K > 8192 || qmax < 1 || M < 0) ? CAMX_EINVAL : CAMX_OK; }

// one instance per number of rounds
#define ACTQ_ROUNDS(K, CALL)                                                                                           \
    switch (((K) + 1023) / 1024) {                                                                                     \
        case 1: { constexpr int NR = 1; CALL; } break; case 2: { constexpr int NR = 2; CALL; } break;                   \
        case 3: { constexpr int NR = 3; CALL; } break; case 4: { constexpr int NR = 4; CALL; } break;                   \
        case 5: { constexpr int NR = 5; CALL; } break; case 6: { constexpr int NR = 6; CALL; } break;                   \
        case 7: { constexpr int NR = 7; CALL; } break; default: { constexpr int NR = 8; CALL; } break;                  \
    }

extern "C" {

// actq_fwd_{f32,bf16} and actq_fwd_codes_{f32,bf16}: y bf16 [M][K] (optional when codes are written), s [M] (optional),
// codes [M][K / 2] bytes (optional; needs qmax <= 7)
int camx_actq_fwd(const void * x, int is_bf16, uint16_t * y, float * s, uint16_t * codes, int K, float clip, int qmax, int M, hipStream_t st) {
    if (!x || (!y && !codes) || actq_check(K, qmax, M) || ((uintptr_t)x & (is_bf16 ? 7 : 15)) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    if (actq_wave_ok(K, x, y, codes)) {
        if (is_bf16) actq_fwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(PlainBF16{(const uint16_t *)x, K}, y, s, codes, K, clip, qmax, M);
        else actq_fwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(PlainF32{(const float *)x, K}, y, s, codes, K, clip, qmax, M);
        CAMX_LAUNCH_RET();
    }
    if (is_bf16) { ACTQ_ROUNDS(K, (actq_fwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(PlainBF16{(const uint16_t *)x, K}, y, s, codes, K, clip, qmax))) }
    else { ACTQ_ROUNDS(K, (actq_fwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(PlainF32{(const float *)x, K}, y, s, codes, K, clip, qmax))) }
    CAMX_LAUNCH_RET();
}
int camx_silu_mul_actq_fwd(const uint16_t * gu, int ld, int F, uint16_t * y, float * s, uint16_t * codes, float clip, int qmax, int M, hipStream_t st) {
    if (!gu || (!y && !codes) || actq_check(F, qmax, M) || ld < 2 * F || (ld & 3) || ((uintptr_t)gu & 7) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    const uint16_t * lut = nullptr, * small = nullptr;
    const int rc = silu_luts_get(st, &lut, &small);
    if (rc) return rc;
    if (F <= 2048 && !(ld & 7) && !((uintptr_t)gu & 15) && actq_wave_ok(F, gu, y, codes)) {       // one wave per row
        actq_fwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(SiluMulSrc{gu, ld, F, lut, nullptr}, y, s, codes, F, clip, qmax, M, small);
        CAMX_LAUNCH_RET();
    }
    ACTQ_ROUNDS(F, (actq_fwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(SiluMulSrc{gu, ld, F, lut, nullptr}, y, s, codes, F, clip, qmax)))
    CAMX_LAUNCH_RET();
}
int camx_block_entry_fwd(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y, float * s, uint16_t * codes,
                         uint16_t * ab, float * rstd_out, int d, float clip, int qmax, int M, hipStream_t st) {
    if (!x || !nw || (!y && !codes) || actq_check(d, qmax, M) || nab < 0 || nab > 16 || (nab && (!wab || !ab)) || ((uintptr_t)x & 15) ||
        ((uintptr_t)nw & 15) || ((uintptr_t)wab & 7) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    if (d <= 1024) {                                     // one wave per row, rounds of 256 values
        switch ((d + 255) / 256) {
            case 1: block_entry_fwd_k<1, 2><<<dim3(M), dim3(64), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax); break;
            case 2: block_entry_fwd_k<2, 2><<<dim3(M), dim3(64), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax); break;
            case 3: block_entry_fwd_k<3, 2><<<dim3(M), dim3(64), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax); break;
            default: block_entry_fwd_k<4, 2><<<dim3(M), dim3(64), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax); break;
        }
        CAMX_LAUNCH_RET();
    }
    ACTQ_ROUNDS(d, (block_entry_fwd_k<NR, 8><<<dim3(M), dim3(256), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax)))
    CAMX_LAUNCH_RET();
}

// actq_bwd_{f32,bf16}: g bf16 [M][K] the gradient of y; dx [M][K] in x's type
int camx_actq_bwd(const void * x, int is_bf16, const uint16_t * g, void * dx, int K, float clip, int qmax, int M, hipStream_t st) {
    if (!x || !g || !dx || actq_check(K, qmax, M) || ((uintptr_t)x & (is_bf16 ? 7 : 15)) || ((uintptr_t)dx & (is_bf16 ? 7 : 15)) || ((uintptr_t)g & 7)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    if (K <= 2048 && !(((uintptr_t)x | (uintptr_t)g | (uintptr_t)dx) & 15)) {                  // one wave per row
        if (is_bf16) actq_bwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(PlainBF16{(const uint16_t *)x, K}, g, SinkBF16{(uint16_t *)dx, K}, K, clip, qmax, M);
        else actq_bwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(PlainF32{(const float *)x, K}, g, SinkF32{(float *)dx, K}, K, clip, qmax, M);
        CAMX_LAUNCH_RET();
    }
    if (is_bf16) { ACTQ_ROUNDS(K, (actq_bwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(PlainBF16{(const uint16_t *)x, K}, g, SinkBF16{(uint16_t *)dx, K}, K, clip, qmax))) }
    else { ACTQ_ROUNDS(K, (actq_bwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(PlainF32{(const float *)x, K}, g, SinkF32{(float *)dx, K}, K, clip, qmax))) }
    CAMX_LAUNCH_RET();
}
// silu_mul_actq_bwd: g bf16 [M][F] the gradient of y; dgu bf16 [M][2F] = [dg | du], contiguous
int camx_silu_mul_actq_bwd(const uint16_t * gu, int ld, int F, const uint16_t * g, uint16_t * dgu, float clip, int qmax, int M, hipStream_t st) {
    if (!gu || !g || !dgu || actq_check(F, qmax, M) || ld < 2 * F || (ld & 3) || ((uintptr_t)gu & 7) || ((uintptr_t)g & 7) || ((uintptr_t)dgu & 7)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    const uint16_t * lut = nullptr, * small = nullptr;
    const float * dlut = nullptr, * dsmall = nullptr;
    int rc = silu_luts_get(st, &lut, &small);
    if (!rc) rc = dsilu_luts_get(st, &dlut, &dsmall);
    if (rc) return rc;
    if (F <= 2048 && !(ld & 7) && !(((uintptr_t)gu | (uintptr_t)g | (uintptr_t)dgu) & 15)) {      // one wave per row
        actq_bwd_wave_k<<<dim3((M + 3) / 4), dim3(256), 0, st>>>(SiluMulSrc{gu, ld, F, lut, nullptr}, g, SinkSiluMul{gu, ld, F, dgu, dlut, nullptr}, F, clip, qmax, M, small, dsmall);
        CAMX_LAUNCH_RET();
    }
    ACTQ_ROUNDS(F, (actq_bwd_k<NR><<<dim3(M), dim3(256), 0, st>>>(SiluMulSrc{gu, ld, F, lut, nullptr}, g, SinkSiluMul{gu, ld, F, dgu, dlut, nullptr}, F, clip, qmax)))
    CAMX_LAUNCH_RET();
}
// block_entry_bwd: dy bf16 [M][d], dab bf16 [M][nab] (needed when nab > 0), rstd [M] from the forward; dx fp32 [M][d]; d <= 1024
int camx_block_entry_bwd(const float * x, const float * nw, const float * rstd, const uint16_t * wab, int nab, const uint16_t * dy,
                         const uint16_t * dab, float * dx, int d, float clip, int qmax, int M, hipStream_t st) {
    if (!x || !nw || !rstd || !dy || !dx || actq_check(d, qmax, M) || d > 1024 || nab < 0 || nab > 16 || (nab & 1) || (nab && (!wab || !dab)) ||
        ((uintptr_t)x & 15) || ((uintptr_t)nw & 15) || ((uintptr_t)dy & 7) || ((uintptr_t)dx & 15) || ((uintptr_t)wab & 7)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    switch ((d + 255) / 256) {
        case 1: block_entry_bwd_k<1><<<dim3(M), dim3(64), 0, st>>>(x, nw, rstd, wab, nab, dy, dab, dx, d, clip, qmax); break;
        case 2: block_entry_bwd_k<2><<<dim3(M), dim3(64), 0, st>>>(x, nw, rstd, wab, nab, dy, dab, dx, d, clip, qmax); break;
        case 3: block_entry_bwd_k<3><<<dim3(M), dim3(64), 0, st>>>(x, nw, rstd, wab, nab, dy, dab, dx, d, clip, qmax); break;
        default: block_entry_bwd_k<4><<<dim3(M), dim3(64), 0, st>>>(x, nw, rstd, wab, nab, dy, dab, dx, d, clip, qmax); break;
    }
    CAMX_LAUNCH_RET();
}

}   // extern "C"
