// Activation quantizers for gfx950: ggml q8_1 blocks (36 B / 32 values) and the MMQ layout (144 B / 128 values), plain,
// behind SwiGLU, and scattered to expert columns. Replaces gg_quantize_q8_1 / OP_GG_Q8_1 (kernels/k3_gguf.hip:29-36,
// kernels/k3_gguf_ops.h:55-77,146-162) and quantize_mmq_q8_1<layout, scatter> (kernels/ggml_mmq/quantize_mmq.cuh:41-140).
//
// Layout of the general q8_1 kernel: 8 lanes x 4 consecutive floats = one 32-value quantization group; a wave covers 256 values
// per step with one 128-bit load per lane. Batches that stream from HBM take a one-lane-per-block kernel (q8_1_blocks) and the
// one-shot MMQ kernel (swiglu_mmq_oneshot), described where they stand.
#include "common.cuh"
#include <mutex>

CAMX_DEV float silu_f(float x) { return x / (1.0f + expf(-x)); }

// ---- q8_1, flat -------------------------------------------------------------------------------------------------------------
// mode 0 plain, 1 silu(x * rs), 2 silu(x) * g[i]; values past n quantize as 0; blocks = ceil(n / 32).
// A wave takes 1024 consecutive values per step: four 128-bit loads per lane issued together, then the 32 blocks (1152
// contiguous bytes) are assembled in the wave's own LDS and leave as 72 aligned 16-byte pieces, instead of 4-byte stores
// that cover each 64-byte line in several partial writes. The last, partial step (and an unaligned y) stores directly.
CAMX_DEV f32x4 q8_1_pre(f32x4 v, f32x4 gv, int mode, float rs, long i0, long n) {
    if (mode == 1) {
        if (i0 + 0 < n) { const float t = v.x * rs; v.x = silu_f(t); }
        if (i0 + 1 < n) { const float t = v.y * rs; v.y = silu_f(t); }
        if (i0 + 2 < n) { const float t = v.z * rs; v.z = silu_f(t); }
        if (i0 + 3 < n) { const float t = v.w * rs; v.w = silu_f(t); }
    } else if (mode == 2) {
        if (i0 + 0 < n) v.x = silu_f(v.x) * gv.x;
        if (i0 + 1 < n) v.y = silu_f(v.y) * gv.y;
        if (i0 + 2 < n) v.z = silu_f(v.z) * gv.z;
        if (i0 + 3 < n) v.w = silu_f(v.w) * gv.w;
    }
    return v;
}
__global__ void __launch_bounds__(256) q8_1_flat(const float * __restrict__ x, uint8_t * __restrict__ y, long n, int mode, float rs,
                                                 const float * __restrict__ g, int vec, int vecst) {
    __shared__ __attribute__((aligned(16))) uint32_t stage[4][288];
    const int lane = slot_of(threadIdx.x & 63), lraw = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const long wave = (long)blockIdx.x * 4 + wv;
    const long nwaves = (long)gridDim.x * 4;
    const long nstep = (n + 1023) >> 10, nb = (n + 31) >> 5;
    f32x4 v[4], gv[4];
    auto load = [&](f32x4 (&v)[4], f32x4 (&gv)[4], long s) {
        const long base = s * 1024;
        if (vec && base + 1024 <= n) {
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = __builtin_nontemporal_load((const f32x4 *)(x + base + 256 * j + 4 * lane));
            if (mode == 2) {
#pragma unroll
                for (int j = 0; j < 4; j++) gv[j] = __builtin_nontemporal_load((const f32x4 *)(g + base + 256 * j + 4 * lane));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const long i0 = base + 256 * j + 4 * lane;
                float t[4] = {0.0f, 0.0f, 0.0f, 0.0f}, tg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int k = 0; k < 4; k++) if (i0 + k < n) { t[k] = x[i0 + k]; if (mode == 2) tg[k] = g[i0 + k]; }
                v[j] = (f32x4){t[0], t[1], t[2], t[3]}; gv[j] = (f32x4){tg[0], tg[1], tg[2], tg[3]};
            }
        }
    };
    for (long s = wave; s < nstep; s += nwaves) {
        const long base = s * 1024;
        load(v, gv, s);
        const bool whole = vecst && s * 32 + 32 <= nb;             // all 32 blocks of the step exist
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const f32x4 q = q8_1_pre(v[j], gv[j], mode, rs, base + 256 * j + 4 * lane, n);
            const long b = s * 32 + 8 * j + (lane >> 3);
            if (whole) {
                const float amax = group8_max(absmax4(q));
                const float sum = group32_sum(q);
                const float d = amax / 127.0f;
                uint32_t codes = 0;
                if (amax != 0.0f) codes = q8_codes4(q, d);
                uint32_t * blk = stage[wv] + (8 * j + (lane >> 3)) * 9;
                blk[1 + (lane & 7)] = codes;
                if ((lane & 7) == 0) blk[0] = (uint32_t)f2h_bits(d) | ((uint32_t)f2h_bits(sum) << 16);
            } else if (b < nb) q8_1_emit(q, y + b * 36, lane & 7);     // (a group of 8 lanes is wholly inside or outside)
        }
        if (whole) {
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_s_waitcnt(0xc07f);                        // lgkmcnt(0): the wave's LDS stores have landed
            u32x4 * dst = (u32x4 *)(y + s * 1152);
            __builtin_nontemporal_store(*(const u32x4 *)(stage[wv] + 4 * lraw), dst + lraw);
            if (lraw < 8) __builtin_nontemporal_store(*(const u32x4 *)(stage[wv] + 4 * (64 + lraw)), dst + 64 + lraw);
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_s_waitcnt(0xc07f);                        // read out before the next step overwrites it
        }
    }
}

// The same blocks for a batch that streams from HBM (modes 0 and 1, whole steps of 2048 values, 16-byte aligned): one lane per
// block. With four values per lane, as above, the eight lanes of a block each repeat the block's divide and walk two
// butterflies, and the vector ALUs, not HBM, set the time. Here a wave's 2048 values go to its own LDS as they arrive (16 bytes
// per lane, neighbouring lanes on neighbouring addresses, no registers held), lane l then quantizes block l whole
// (q8_1_block_lane: everything per block happens once, same sum tree), and the blocks leave as 16-byte stores.
template <int MODE>
__global__ void __launch_bounds__(256) q8_1_blocks(const float * __restrict__ x, uint8_t * __restrict__ y, float rs) {
    __shared__ __attribute__((aligned(16))) float in_all[4][2048];
    __shared__ __attribute__((aligned(16))) uint32_t stage_all[4][576];
    const int l = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t step = (size_t)blockIdx.x * 4 + wv;
    float * in = in_all[wv];
    uint32_t * stage = stage_all[wv];
    const float * src = x + step * 2048;
#pragma unroll
    for (int i = 0; i < 8; i++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + 256 * i + 4 * l), (__attribute__((address_space(3))) void *)(in + 256 * i), 16, 0, 2);
    __builtin_amdgcn_s_waitcnt(0x0f70);                                    // vmcnt(0): the wave's own values have landed
    q8_1_block_lane<MODE>(in + 32 * l, stage + 9 * l, l, rs);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();       // the wave's own LDS writes, in order
    u32x4 * dst = (u32x4 *)(y + step * 2304);
    __builtin_nontemporal_store(*(const u32x4 *)(stage + 4 * l), dst + l);
    __builtin_nontemporal_store(*(const u32x4 *)(stage + 4 * (64 + l)), dst + 64 + l);
    if (l < 16) __builtin_nontemporal_store(*(const u32x4 *)(stage + 4 * (128 + l)), dst + 128 + l);
}

// ---- q8_1 in the MMQ layout ---------------------------------------------------------------------------------------------------
enum { MMQ_D4 = 0, MMQ_DS4 = 1 };
enum { SRC_F32 = 0, SRC_SWIGLU_BF16 = 1 };

struct MmqArgs {
    const void * x;          // SRC_F32: fp32 rows; SRC_SWIGLU_BF16: bf16 rows [g | u], F = K
    const int32_t * ids;     // gather: source row of column c (null: c); scatter: destination columns [ntok][k]
    uint8_t * y;             // [Kp / 128][ncols] blocks of 144 B
    uint16_t * act;          // SRC_SWIGLU_BF16 only, optional: the bf16 activation [ncols_src][K]
    long K, Kp, stride;      // values per row, padded to 512, source row stride in elements
    int ncols;               // destination columns
    int nsrc;                // source rows the grid walks (ncols, or ntok when scattering)
    int kexp;                // scatter: destination columns per source row (0: no scatter)
    const uint16_t * lut;    // SRC_SWIGLU_BF16: the table of bf16(silu g) in device memory
};

CAMX_DEV f32x4 swiglu_bf16x4(u32x2 gw, u32x2 uw, u32x2 * packed, const uint16_t * __restrict__ lut) {
    const f32x4 u = unpack_bf16x4(uw);
    f32x4 a;
    a.x = bf2f(lut[gw.x & 0xffffu]) * u.x; a.y = bf2f(lut[gw.x >> 16]) * u.y;
    a.z = bf2f(lut[gw.y & 0xffffu]) * u.z; a.w = bf2f(lut[gw.y >> 16]) * u.w;
    const u32x2 p = pack_f2bf_x4(a);
    *packed = p;
    return unpack_bf16x4(p);
}

template <int LAYOUT, int SRC>
__global__ void __launch_bounds__(256) mmq_q8_1_rows(MmqArgs a) {
    const int lane = slot_of(threadIdx.x & 63);
    // Scattering: workgroups are dealt to the eight XCDs in turn, and each XCD has its own L2. A token's 144-byte blocks share their
    // 128-byte lines with the blocks of the neighbouring columns, which belong to tokens a few rows away (the router groups columns by
    // expert, a group's tokens in order); when those tokens run on another XCD the two halves of a line leave as two partial writes.
    // So an XCD takes a contiguous range of token groups (workgroup b -> group (b % 8) * (G / 8) + b / 8), and neighbours meet in one L2.
    int bx = blockIdx.x;
    if (a.kexp && (gridDim.x & 7) == 0) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);
    const int col = bx * 4 + (threadIdx.x >> 6);                    // source row index
    if (col >= a.nsrc) return;
    const long slab = blockIdx.y;                                   // 256 values = 2 blocks of 128
    const long i0 = slab * 256 + 4 * lane;
    if (i0 >= a.Kp) return;                                         // (Kp is a multiple of 512: never taken for half a wave)
    const long srow = a.kexp ? col : (a.ids ? a.ids[col] : col);
    // scattering: the row's destination columns come in with the row (lane s holds column s of each batch of 64), not one dependent
    // load per column between the stores
    const int lraw = threadIdx.x & 63;
    int dcols = 0;
    if (a.kexp && lraw < a.kexp) dcols = a.ids[(long)col * a.kexp + lraw];
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i0 < a.K) {                                                 // K % 4 == 0: a lane's four values are in or out together
        if (SRC == SRC_F32) v = *(const f32x4 *)((const float *)a.x + srow * a.stride + i0);
        else {
            const uint16_t * r = (const uint16_t *)a.x + srow * a.stride;
            u32x2 packed;
            v = swiglu_bf16x4(*(const u32x2 *)(r + i0), *(const u32x2 *)(r + a.K + i0), &packed, a.lut);
            if (a.act) *(u32x2 *)(a.act + srow * a.K + i0) = packed;
        }
    }
    float amax = group8_max(absmax4(v));
    float sum = 0.0f;
    if (LAYOUT == MMQ_DS4) sum = group8_sum(((v.x + v.y) + v.z) + v.w);
    uint32_t q = 0; float d = 0.0f;
    if (amax != 0.0f) {
        const float d_inv = 127.0f / amax;
        f32x4 t; t.x = v.x * d_inv; t.y = v.y * d_inv; t.z = v.z * d_inv; t.w = v.w * d_inv;
        q = pack_round_i8x4(t);
        d = 1.0f / d_inv;
    }
    const long kb = slab * 2 + (lane >> 5);
    const int l32 = lane & 31;
    const uint32_t hdr = LAYOUT == MMQ_DS4 ? ((uint32_t)f2h_bits(d) | ((uint32_t)f2h_bits(sum) << 16)) : __builtin_bit_cast(uint32_t, d);
    const int nwrite = a.kexp ? a.kexp : 1;
    for (int slot = 0; slot < nwrite; slot++) {
        if (a.kexp && slot >= 64 && (slot & 63) == 0) dcols = slot + lraw < a.kexp ? a.ids[(long)col * a.kexp + slot + lraw] : 0;
        const long dcol = a.kexp ? __builtin_amdgcn_readlane(dcols, slot & 63) : col;
        uint8_t * blk = a.y + (kb * a.ncols + dcol) * 144;
        *(uint32_t *)(blk + 16 + 4 * l32) = q;
        if ((lane & 7) == 0) *(uint32_t *)(blk + 4 * (l32 >> 3)) = hdr;
    }
}

template <int SRC>
static int launch_mmq(const MmqArgs & a, int layout, hipStream_t st) {
    if (a.nsrc <= 0) return CAMX_OK;
    const dim3 grid((a.nsrc + 3) / 4, (unsigned)(a.Kp / 256)), block(256);
    if (layout == MMQ_DS4) mmq_q8_1_rows<MMQ_DS4, SRC><<<grid, block, 0, st>>>(a);
    else mmq_q8_1_rows<MMQ_D4, SRC><<<grid, block, 0, st>>>(a);
    CAMX_LAUNCH_RET();
}

// ---- fused SwiGLU -> MMQ q8_1, the wide form ---------------------------------------------------------------------------------
// bf16(silu(g)) of a bf16 g is a function of 16 bits: the whole table (65536 x 2 B = 128 KiB) fits in one CU's 160 KiB of
// LDS. Persistent workgroups (one per CU, 16 waves) copy the table from a static device array once and then look every
// gate value up with one 16-bit LDS read, which takes the two transcendentals, the divide and the first bf16 rounding
// off the VALU. The table itself is computed once per device ((float)exp in double, then the reference's fp32 statement
// g / (1 + e), then round-to-nearest-even to bf16).
//
// A wave's work item is 8 tokens x one 128-value block column: lane l takes the 8 consecutive values 8 (l & 15) .. + 7 of
// tokens (l >> 4) and (l >> 4) + 4 (load i = token half i), so that one 128-bit load instruction of g (and of u) fetches
// four 256-byte row pieces. Items are numbered with the token group running fastest inside a band of four block columns,
// so the waves that run together read different rows (1 KiB of each) and write four long runs of blocks. A 32-value
// quantization group is the 4 lanes of a quad (for each i), a 128-value block 16 lanes. The reference's
// 8 threads of a group are (lane & 3, half): thread 2 (lane & 3) + h holds values 4h .. 4h + 3 of the lane, so its
// xor 4 / 2 / 1 butterfly is lane ^ 2, lane ^ 1 (quad permutes) and the lane's two halves. Lane (l & 3) == i does
// group i's two IEEE divisions (127 / amax, 1 / d_inv); the quad reads d_inv back through a DPP broadcast.
//
// Output: the 144-byte blocks of the item's 8 tokens are contiguous in the block row (1152 B = 9 whole 128-byte lines).
// Written straight from the lanes they would leave as 8-byte pieces that straddle 64-byte boundaries (3.3 write requests
// per block instead of 2.25, each costing a full 64-byte slot on the way to HBM), so a wave stages its blocks in its own
// 1152 bytes of LDS and writes them out as one aligned run of 16 bytes per lane. Nothing but the table is shared
// between waves: no barrier after the table copy, every wave runs its own pipeline (two items of loads in flight).
#define SWM_TOK 8
#define SWM_STAGE (16 * SWM_TOK * 144)           // 16 waves x 1152 bytes
#define SWM_LDS (131072 + SWM_STAGE)

__device__ uint16_t g_silu_lut[65536];
__device__ __attribute__((aligned(16))) uint32_t g_zero16[4] = {0, 0, 0, 0};   // (not const: it must live in the global address space, or the selects below turn the loads into flat ones)

__global__ void __launch_bounds__(256) silu_lut_fill() {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    const float g = bf2f((uint16_t)i);
    const float e = (float)exp(-(double)g);          // the correctly rounded expf(-g)
    g_silu_lut[i] = f2bf(g / (1.0f + e));
}

CAMX_DEV uint32_t cvt_pk_bf16(float lo, float hi) { return hw_pk_bf16(lo, hi); }
CAMX_DEV int round_i32(float v) { return (int)(v + __builtin_copysignf(0.49999997f, v)); }
CAMX_DEV uint32_t pack_i8x4(int q0, int q1, int q2, int q3) {
    return __builtin_amdgcn_perm((uint32_t)q1, (uint32_t)q0, 0x0c0c0400u) | __builtin_amdgcn_perm((uint32_t)q3, (uint32_t)q2, 0x04000c0cu);
}
template <int I> CAMX_DEV float quad_bcast(float v) {     // every lane of a quad gets lane I's value
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), I * 0x55, 0xf, 0xf, false));
}
CAMX_DEV float max3_abs(float a, float b, float c) { return fmaxf(fmaxf(fabsf(a), fabsf(b)), c); }

struct SwmItem { u32x4 gw[2], uw[2]; };

// issue the four 128-bit loads of work item (tokens tg .. tg + 7, block column unit). Every lane always issues all four
// (a lane past the row's end or past the last token, or a whole wave without work, reads 16 zero bytes instead): with a
// fixed number of loads in flight the compiler can wait for exactly the older item's data and leave this item's loads
// outstanding across the other item's arithmetic.
template <int SRC>
CAMX_DEV void swm_load(SwmItem & it, const void * __restrict__ src, const int32_t * __restrict__ ids, long ld, long F, int T, long tg, long unit,
                       int lane, bool valid) {
    const long e0 = unit * 128 + 8 * (lane & 15);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const long t = tg + (lane >> 4) + 4 * i;
        const bool tok = valid && t < T;
        if (SRC == SRC_SWIGLU_BF16) {
            const bool ok = tok && e0 < F;
            const uint16_t * r = (const uint16_t *)src + (size_t)(ok ? t : 0) * ld + e0;
            const u32x4 * pg = ok ? (const u32x4 *)r : (const u32x4 *)g_zero16;
            const u32x4 * pu = ok ? (const u32x4 *)(r + F) : (const u32x4 *)g_zero16;
            it.gw[i] = __builtin_nontemporal_load(pg); it.uw[i] = __builtin_nontemporal_load(pu);     // read once, never written: +15 % over plain loads
        } else {                                                // fp32 rows: gw[i] = values 0 .. 3, uw[i] = values 4 .. 7 of the lane's eight
            const long row = tok ? (ids ? ids[t] : t) : 0;
            const float * r = (const float *)src + (size_t)row * ld + e0;
            const u32x4 * p0 = tok && e0 < F ? (const u32x4 *)r : (const u32x4 *)g_zero16;
            const u32x4 * p1 = tok && e0 + 4 < F ? (const u32x4 *)(r + 4) : (const u32x4 *)g_zero16;
            it.gw[i] = __builtin_nontemporal_load(p0); it.uw[i] = __builtin_nontemporal_load(p1);
        }
    }
}

// the item's arithmetic; the wave's 8 blocks go to stage[token slot][144] (the wave's own 1152 bytes)
// CANON: the activation is packed with f2bf (a NaN becomes 0x7fc0, as silu_mul_bf16 stores it) instead of the hardware convert, which
// keeps a NaN's sign and payload. Returns whether a group sum of this lane's quad is a NaN: the callers run the item with the hardware
// convert first and, in the rare wave that reports one (a NaN or infinite input), once more with CANON, which rewrites the same bytes.
// LUTMODE: where bf16(silu g) comes from. LUT_FULL: the 65536-entry table (in LDS for the persistent kernel, in device memory for the
// rare redo of the one-shot kernel). LUT_SMALL: the 8192-entry table of the one-shot kernel, which holds the gates a model produces
// (+-0 and 2^-24 <= |g| < 2^8 less two values); bit 1 of the result reports a gate outside it, and the caller redoes the item with the full table.
enum { LUT_FULL = 0, LUT_SMALL = 1 };
template <int LAYOUT, int SRC, bool CANON = false, int LUTMODE = LUT_FULL>
CAMX_DEV int swm_compute(const SwmItem & it, const uint16_t * lut, uint8_t * stage, long F, uint16_t * __restrict__ act, int T, long tg, long unit,
                         int lane) {
    const int lq = lane & 3;
    const long e0 = unit * 128 + 8 * (lane & 15);
    float val[2][8];                                                   // the lane's eight values of each half, as quantized
    float amax[2], sum[2];
    u16x2 gmin = {0xffff, 0xffff}, gmax = {0, 0};                      // LUT_SMALL: min of |g| - 1 (a zero wraps to 0xffff), max of |g|, per half
#pragma unroll
    for (int i = 0; i < 2; i++) {
        float m = 0.0f, s0 = 0.0f, s1 = 0.0f;
        uint32_t pk[4];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            float v0, v1;
            if (SRC == SRC_SWIGLU_BF16) {
                uint32_t sl, sh;
                if (LUTMODE == LUT_SMALL) {
                    const uint32_t w = it.gw[i][p];
                    const u16x2 a2 = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
                    const u16x2 i2 = __builtin_elementwise_min(a2 - (u16x2){SWS_A0, SWS_A0}, (u16x2){SWS_SPAN, SWS_SPAN});      // below the table: wraps, clamps
                    const uint32_t idx = ((w >> 3) & 0x10001000u) | __builtin_bit_cast(uint32_t, i2);                            // the sign in bit 12
                    gmin = __builtin_elementwise_min(gmin, a2 - (u16x2){1, 1}); gmax = __builtin_elementwise_max(gmax, a2);
                    sl = lut[idx & 0xffffu]; sh = lut[idx >> 16];
                } else { sl = lut[it.gw[i][p] & 0xffffu]; sh = lut[it.gw[i][p] >> 16]; }
                const float u0 = __builtin_bit_cast(float, it.uw[i][p] << 16), u1 = __builtin_bit_cast(float, it.uw[i][p] & 0xffff0000u);
                const float a0 = __builtin_bit_cast(float, sl << 16) * u0, a1 = __builtin_bit_cast(float, sh << 16) * u1;
                pk[p] = CANON ? ((uint32_t)f2bf(a0) | ((uint32_t)f2bf(a1) << 16)) : cvt_pk_bf16(a0, a1);
                v0 = __builtin_bit_cast(float, pk[p] << 16); v1 = __builtin_bit_cast(float, pk[p] & 0xffff0000u);
            } else {
                const u32x4 w = p < 2 ? it.gw[i] : it.uw[i];
                const uint32_t b0 = w[2 * (p & 1)], b1 = w[2 * (p & 1) + 1];     // (a bit cast applied straight to a vector element reads element 0)
                v0 = __builtin_bit_cast(float, b0); v1 = __builtin_bit_cast(float, b1);
            }
            val[i][2 * p] = v0; val[i][2 * p + 1] = v1;
            m = max3_abs(v0, v1, m);
            if (LAYOUT == MMQ_DS4 || SRC == SRC_SWIGLU_BF16) {      // per thread ((x0 + x1) + x2) + x3: pairs p = 0, 1 are thread h = 0, pairs 2, 3 thread h = 1 (the bf16 source keeps the sums in the D4 layout too: a NaN shows in them)
                if (p == 0) s0 = v0 + v1; else if (p == 1) s0 = (s0 + v0) + v1; else if (p == 2) s1 = v0 + v1; else s1 = (s1 + v0) + v1;
            }
        }
        const long t = tg + (lane >> 4) + 4 * i;
        if (SRC == SRC_SWIGLU_BF16 && act && t < T && e0 < F) *(u32x4 *)(act + (size_t)t * F + e0) = (u32x4){pk[0], pk[1], pk[2], pk[3]};
        m = fmaxf(m, lane_xor2(m)); amax[i] = fmaxf(m, lane_xor1(m));
        sum[i] = 0.0f;
        if (LAYOUT == MMQ_DS4 || SRC == SRC_SWIGLU_BF16) {
            s0 += lane_xor2(s0); s1 += lane_xor2(s1);          // thread ^ 4
            s0 += lane_xor1(s0); s1 += lane_xor1(s1);          // thread ^ 2
            sum[i] = s0 + s1;                                   // thread ^ 1
        }
    }
    // lanes 0 and 1 of a quad own the quad's two groups (lanes 2, 3 repeat group 1's division; their header is not stored)
    const int own = lq & 1;
    const float am = own ? amax[1] : amax[0], sm = own ? sum[1] : sum[0];
    float d_inv = 0.0f, d = 0.0f;
    if (am != 0.0f) { d_inv = 127.0f / am; d = 1.0f / d_inv; }
    const float di[2] = {quad_bcast<0>(d_inv), quad_bcast<1>(d_inv)};
    uint8_t * blk0 = stage + (lane >> 4) * 144;                            // token slot (lane >> 4) + 4 i
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int q[8];
#pragma unroll
        for (int p = 0; p < 8; p++) q[p] = round_i32(val[i][p] * di[i]);
        *(u32x2 *)(blk0 + i * (4 * 144) + 16 + 8 * (lane & 15)) = (u32x2){pack_i8x4(q[0], q[1], q[2], q[3]), pack_i8x4(q[4], q[5], q[6], q[7])};
    }
    if (lq < 2)
        *(uint32_t *)(blk0 + lq * (4 * 144) + 4 * ((lane & 15) >> 2)) =
            LAYOUT == MMQ_DS4 ? ((uint32_t)f2h_bits(d) | ((uint32_t)f2h_bits(sm) << 16)) : __builtin_bit_cast(uint32_t, d);
    int flags = SRC == SRC_SWIGLU_BF16 && !CANON && ((sum[0] != sum[0]) | (sum[1] != sum[1]));
    if (LUTMODE == LUT_SMALL)
        flags |= ((gmin.x < SWS_A0 - 1) | (gmin.y < SWS_A0 - 1) | (gmax.x >= SWS_A0 + SWS_SPAN) | (gmax.y >= SWS_A0 + SWS_SPAN)) ? 2 : 0;
    return flags;
}

// SRC_F32 (quantize_mmq_q8_1 without scatter): the same work split and copy-out on fp32 rows (column c = row ids[c] or c), no table
template <int LAYOUT, int SRC>
__global__ void __launch_bounds__(1024) swiglu_mmq_lut(const void * __restrict__ gu, const int32_t * __restrict__ ids, long ld, long F,
                                                       uint8_t * __restrict__ y, uint16_t * __restrict__ act, int T, unsigned ncol, unsigned nitems) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t * stage = (uint8_t *)lut + (SRC == SRC_SWIGLU_BF16 ? 131072 : 0) + wave * (SWM_TOK * 144);
    const unsigned stride = gridDim.x * 16;                                   // (ids stay below 2^31: checked by the launcher)
    unsigned j = blockIdx.x * 16 + wave;
    // item id -> 4 neighbouring block columns x token groups, token groups fastest: the four waves of a SIMD row read 1 KiB of each token row
    // and the workgroups that run side by side write neighbouring runs of the same block rows (ncol is a multiple of 4: K is padded to 512)
    const unsigned ntg = (unsigned)((T + SWM_TOK - 1) / SWM_TOK);
#define SWM_TG(id) ((long)((((id) >> 2) % ntg)) * SWM_TOK)
#define SWM_UNIT(id) ((long)(((((id) >> 2) / ntg) << 2) + ((id) & 3)))
    SwmItem A, B, C;                                                          // three items in rotation: two steps of loads in flight
    swm_load<SRC>(A, gu, ids, ld, F, T, SWM_TG(j), SWM_UNIT(j), lane, j < nitems);                  // in flight while the table is copied
    swm_load<SRC>(B, gu, ids, ld, F, T, SWM_TG(j + stride), SWM_UNIT(j + stride), lane, j + stride < nitems);
    if (SRC == SRC_SWIGLU_BF16) {
        for (int i = threadIdx.x; i < 8192; i += 1024) ((u32x4 *)lut)[i] = ((const u32x4 *)g_silu_lut)[i];
        __syncthreads();
    }
    // copy-out of a finished item: 1152 contiguous bytes = 72 lanes' worth of 16 B (lanes 0 .. 7 take a second unit)
    auto flush = [&](unsigned id) {
        const long tg = SWM_TG(id), unit = SWM_UNIT(id);
        const int nunits = (int)min((long)SWM_TOK, T - tg) * 9;               // tokens of the group that exist
        uint8_t * dst = y + ((size_t)unit * T + (size_t)tg) * 144;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();       // the wave's own LDS writes, in order
        if (lane < nunits) __builtin_nontemporal_store(*(const u32x4 *)(stage + 16 * lane), (u32x4 *)(dst + 16 * lane));
        if (lane < 8 && 64 + lane < nunits) __builtin_nontemporal_store(*(const u32x4 *)(stage + 1024 + 16 * lane), (u32x4 *)(dst + 1024 + 16 * lane));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
    };
#define SWM_STEP(CUR, NXT2, jc)                                                                                              \
    {                                                                                                                        \
        const unsigned jn = (jc) + 2 * stride;                                                                                  \
        swm_load<SRC>(NXT2, gu, ids, ld, F, T, SWM_TG(jn), SWM_UNIT(jn), lane, jn < nitems);                                 \
        if ((jc) < nitems) {                                                                                                 \
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(swm_compute<LAYOUT, SRC>(CUR, lut, stage, F, act, T, SWM_TG(jc), SWM_UNIT(jc), lane) & 1) != 0, 0))  \
                swm_compute<LAYOUT, SRC, true>(CUR, lut, stage, F, act, T, SWM_TG(jc), SWM_UNIT(jc), lane);                  \
            flush(jc);                                                                                                       \
        }                                                                                                                    \
    }
    for (; j < nitems; j += 3 * stride) {
        SWM_STEP(A, C, j)
        SWM_STEP(B, A, j + stride)
        SWM_STEP(C, B, j + 2 * stride)
    }
#undef SWM_STEP
#undef SWM_TG
#undef SWM_UNIT
}

// ---- the one-shot form for prefill chunks -----------------------------------------------------------------------------------------
// A workgroup of SWS_WAVES waves takes SWS_WAVES neighbouring token groups of one block column and ends; the hardware hands the next
// workgroup to whichever CU is free, which keeps the chip's accesses inside a narrow moving window of the inputs and makes neighbouring
// waves write neighbouring runs of one block row (measured with every launch on cold lines, the same access pattern runs 12 % faster
// than under persistent workgroups). Several workgroups share a CU, so the table they look gates up in must be small: the 8192
// entries that cover +-0 and 2^-24 <= |g| < 2^8 (16 KiB, copied straight from device memory into LDS, no registers), index = the
// magnitude's offset from 2^-24 clamped to the last entry, which holds +-0. A wave that meets a gate outside the table (2 in the
// flags) redoes its item with the full table in device memory; one that meets a NaN redoes it with the canonical NaN.
#define SWS_WAVES 4
__device__ __attribute__((aligned(16))) uint16_t g_silu_small[SWS_TAB];

__global__ void __launch_bounds__(256) silu_small_fill() {             // after silu_lut_fill, on the same stream
    const uint32_t e = blockIdx.x * 256 + threadIdx.x;
    if (e >= SWS_TAB) return;
    const uint32_t sign = e >> 12, i = e & SWS_SPAN;
    g_silu_small[e] = i == SWS_SPAN ? (uint16_t)(sign << 15) : g_silu_lut[(sign << 15) | (SWS_A0 + i)];
}

#define SWS_IPW 2                                                          // items (token groups) per wave, loaded together
// SCAT (quantize_mmq_q8_1's scatter form): row t is token t, and each of its blocks goes to the kexp columns sc_ids[t * kexp + slot] of a
// block row of ncols_dst columns: the group's eight staged blocks leave as 16-byte pieces, 8 kexp block copies per item (the rows kernel
// writes the same blocks four bytes per lane, two blocks per wave: 35 against 23 us for 4096 tokens x 2048 to 8 columns each).
template <int LAYOUT, int SRC, bool SCAT = false>
__global__ void __launch_bounds__(SWS_WAVES * 64) swiglu_mmq_oneshot(const void * __restrict__ gu, const int32_t * __restrict__ ids, long ld, long F,
                                                                    uint8_t * __restrict__ y, uint16_t * __restrict__ act, int T, unsigned ncolp,
                                                                    const int32_t * __restrict__ sc_ids = nullptr, int kexp = 0, int ncols_dst = 0) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    const int lraw = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t * stage = (uint8_t *)lut + (SRC == SRC_SWIGLU_BF16 ? 2 * SWS_TAB : 0) + wave * (SWM_TOK * 144);
    if (SRC == SRC_SWIGLU_BF16) {
#pragma unroll
        for (int j = wave; j < 2 * SWS_TAB / 1024; j += SWS_WAVES)        // the table, 1 KiB per wave instruction
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(g_silu_small + 512 * j + 8 * lraw),
                                             (__attribute__((address_space(3))) void *)(lut + 512 * j), 16, 0, 0);
    }
    const unsigned ntb = gridDim.x / ncolp;                              // workgroups walk the token groups of a block column first
    // the block column moves on by one every 16 workgroups (1024 tokens) of the walk: with a row stride that is a power of two (8192
    // fp32 values) the rows of one column fall on a fraction of the memory channels, and the walk would keep the whole chip on them
    // (8192 x 8192: 0.60 -> 0.72 of peak; 6144- and 17408-wide rows: unchanged)
    unsigned tb = blockIdx.x % ntb, un = blockIdx.x / ntb + tb / 16;
    if (SCAT && (ntb & 7) == 0) {
        // Scattering: a block shares its first and last line with the blocks of the neighbouring columns, which belong to tokens a few rows
        // away (the router groups columns by expert, a group's tokens in order). Workgroups are dealt to the eight XCDs in turn and each
        // XCD has its own L2, so an XCD takes a contiguous eighth of the token blocks: neighbours meet in one L2 and leave as whole lines.
        const unsigned m = blockIdx.x >> 3, per = ntb >> 3;
        tb = (blockIdx.x & 7) * per + m % per; un = m / per;
    }
    const long tg0 = ((long)tb * SWS_WAVES + wave) * (SWM_TOK * SWS_IPW), unit = un % ncolp;
    SwmItem it[SWS_IPW];
    if (SRC == SRC_F32) {
        // fp32 rows: a lane's eight values are 32 bytes, so loading them into its registers takes two requests that each use half of
        // every line. The rows go to LDS instead, 16 bytes per lane with neighbouring lanes on neighbouring addresses (one request
        // per line, no registers held while they fly), and each lane then reads its eight values from there.
        float * in = (float *)((uint8_t *)lut + SWS_WAVES * (SWM_TOK * 144)) + wave * (SWS_IPW * SWM_TOK * 128);
#pragma unroll
        for (int k = 0; k < SWS_IPW; k++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const long t = tg0 + SWM_TOK * k + 2 * i + (lraw >> 5), e = unit * 128 + 4 * (lraw & 31);
                const bool ok = t < T && e < F;
                const float * p = ok ? (const float *)gu + (size_t)(ids ? ids[t] : t) * ld + e : (const float *)g_zero16;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                                 (__attribute__((address_space(3))) void *)(in + k * (SWM_TOK * 128) + i * 256), 16, 0, 2);
            }
        __builtin_amdgcn_s_waitcnt(0x0f70);                               // vmcnt(0): the wave's own rows have landed
#pragma unroll
        for (int k = 0; k < SWS_IPW; k++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const float * q = in + k * (SWM_TOK * 128) + ((lraw >> 4) + 4 * i) * 128 + 8 * (lraw & 15);
                it[k].gw[i] = *(const u32x4 *)q; it[k].uw[i] = *(const u32x4 *)(q + 4);
            }
    } else {
#pragma unroll
        for (int k = 0; k < SWS_IPW; k++) swm_load<SRC>(it[k], gu, ids, ld, F, T, tg0 + SWM_TOK * k, unit, lraw, tg0 + SWM_TOK * k < T);
        __builtin_amdgcn_s_waitcnt(0x0f70);                               // vmcnt(0): this wave's part of the table has landed (and its items)
        __syncthreads();
    }
#pragma unroll
    for (int k = 0; k < SWS_IPW; k++) {
        const long tg = tg0 + SWM_TOK * k;
        if (tg >= T) return;
        int fl = swm_compute<LAYOUT, SRC, false, SRC == SRC_SWIGLU_BF16 ? LUT_SMALL : LUT_FULL>(it[k], lut, stage, F, act, T, tg, unit, lraw);
        if (SRC == SRC_SWIGLU_BF16) {
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(fl & 2) != 0, 0))
                fl = swm_compute<LAYOUT, SRC, false, LUT_FULL>(it[k], g_silu_lut, stage, F, act, T, tg, unit, lraw);
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(fl & 1) != 0, 0))
                swm_compute<LAYOUT, SRC, true, LUT_FULL>(it[k], g_silu_lut, stage, F, act, T, tg, unit, lraw);
        }
        const int nunits = (int)min((long)SWM_TOK, T - tg) * 9;           // tokens of the group that exist
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();       // the wave's own LDS writes, in order
        if (SCAT) {
            const int nbc = (nunits / 9) * kexp;                          // block copies of the group: token slot b / kexp to its column number b % kexp
            for (int b0 = 0; b0 < nbc; b0 += 64) {
                const int dc = b0 + lraw < nbc ? sc_ids[(size_t)tg * kexp + b0 + lraw] : 0;        // (the group's columns are one contiguous run of the list)
                const int nb = nbc - b0 < 64 ? nbc - b0 : 64;
#pragma unroll
                for (int i = 0; i < 9; i++) {
                    const int p = 64 * i + lraw, b = p / 9, part = p - 9 * b;
                    const int col = __shfl(dc, b & 63, 64);
                    // (plain stores: a block shares its first and last line with the neighbouring columns' blocks, which other workgroups write;
                    // the lines are completed in L2. Past the caches each block would leave as partial lines: 51 instead of 25 us)
                    if (b < nb) *(u32x4 *)(y + ((size_t)unit * ncols_dst + col) * 144 + 16 * part) = *(const u32x4 *)(stage + ((b0 + b) / kexp) * 144 + 16 * part);
                }
            }
        } else {
            uint8_t * dst = y + ((size_t)unit * T + (size_t)tg) * 144;
            if (lraw < nunits) __builtin_nontemporal_store(*(const u32x4 *)(stage + 16 * lraw), (u32x4 *)(dst + 16 * lraw));
            if (lraw < 8 && 64 + lraw < nunits) __builtin_nontemporal_store(*(const u32x4 *)(stage + 1024 + 16 * lraw), (u32x4 *)(dst + 1024 + 16 * lraw));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
    }
}
template <int SRC>
static void launch_oneshot(const void * src, const int32_t * ids, long ld, long F, void * vy, uint16_t * act, int T, long ncol, int layout, hipStream_t st) {
    const int per = SWS_WAVES * SWM_TOK * SWS_IPW;
    const dim3 grid((unsigned)((T + per - 1) / per) * (unsigned)ncol), block(SWS_WAVES * 64);
    const size_t lds = (SRC == SRC_SWIGLU_BF16 ? 2 * SWS_TAB : SWS_WAVES * SWS_IPW * SWM_TOK * 512) + SWS_WAVES * SWM_TOK * 144;
    if (layout == MMQ_DS4) swiglu_mmq_oneshot<MMQ_DS4, SRC><<<grid, block, lds, st>>>(src, ids, ld, F, (uint8_t *)vy, act, T, (unsigned)ncol);
    else swiglu_mmq_oneshot<MMQ_D4, SRC><<<grid, block, lds, st>>>(src, ids, ld, F, (uint8_t *)vy, act, T, (unsigned)ncol);
}
static void launch_oneshot_scatter(const float * x, const int32_t * sc_ids, long ld, long K, void * vy, int ntok, int kexp, int ncols_dst, long ncol, int layout, hipStream_t st) {
    const int per = SWS_WAVES * SWM_TOK * SWS_IPW;
    const dim3 grid((unsigned)((ntok + per - 1) / per) * (unsigned)ncol), block(SWS_WAVES * 64);
    const size_t lds = SWS_WAVES * SWS_IPW * SWM_TOK * 512 + SWS_WAVES * SWM_TOK * 144;
    if (layout == MMQ_DS4) swiglu_mmq_oneshot<MMQ_DS4, SRC_F32, true><<<grid, block, lds, st>>>(x, nullptr, ld, K, (uint8_t *)vy, nullptr, ntok, (unsigned)ncol, sc_ids, kexp, ncols_dst);
    else swiglu_mmq_oneshot<MMQ_D4, SRC_F32, true><<<grid, block, lds, st>>>(x, nullptr, ld, K, (uint8_t *)vy, nullptr, ntok, (unsigned)ncol, sc_ids, kexp, ncols_dst);
}

// act = bf16(bf16(silu g) * u) of wide bf16 rows [g (H) | u (H)] with the same table: persistent workgroups, a lane takes 8
// values at a time (16 bytes of g, of u, of act) and keeps the next unit's loads in flight across the current one's lookups.
// The products are rounded by the packed hardware convert; a unit that holds a NaN is redone with the canonical NaN.
__global__ void __launch_bounds__(1024) silu_mul_lut(const uint16_t * __restrict__ gu, uint16_t * __restrict__ act, unsigned H8, unsigned n8) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    const unsigned S = gridDim.x * 1024u, dr = S / H8, dc = S % H8;
    unsigned q = blockIdx.x * 1024u + threadIdx.x, r = q / H8, c = q % H8;
    auto addr = [&](bool ok) { return ok ? (const u32x4 *)(gu + ((size_t)r * 2 * H8 + c) * 8) : (const u32x4 *)g_zero16; };
    const u32x4 * p = addr(q < n8);
    u32x4 g = __builtin_nontemporal_load(p), u = __builtin_nontemporal_load(q < n8 ? p + H8 : p);
    for (unsigned i = threadIdx.x; i < 8192; i += 1024) ((u32x4 *)lut)[i] = ((const u32x4 *)g_silu_lut)[i];
    __syncthreads();
    while (q < n8) {
        const size_t o = ((size_t)r * H8 + c) * 8;
        const unsigned qn = q + S;
        c += dc; r += dr;
        if (c >= H8) { c -= H8; r++; }
        const u32x4 * pn = addr(qn < n8);
        const u32x4 gn = __builtin_nontemporal_load(pn), un = __builtin_nontemporal_load(qn < n8 ? pn + H8 : pn);
        uint32_t pk[4];
        bool nan = false;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t gw = g[k], uw = u[k];
            const float a0 = __builtin_bit_cast(float, (uint32_t)lut[gw & 0xffffu] << 16) * __builtin_bit_cast(float, uw << 16);
            const float a1 = __builtin_bit_cast(float, (uint32_t)lut[gw >> 16] << 16) * __builtin_bit_cast(float, uw & 0xffff0000u);
            nan |= (a0 != a0) | (a1 != a1);
            pk[k] = cvt_pk_bf16(a0, a1);
        }
        if (nan) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t gw = g[k], uw = u[k];
                const float a0 = __builtin_bit_cast(float, (uint32_t)lut[gw & 0xffffu] << 16) * __builtin_bit_cast(float, uw << 16);
                const float a1 = __builtin_bit_cast(float, (uint32_t)lut[gw >> 16] << 16) * __builtin_bit_cast(float, uw & 0xffff0000u);
                pk[k] = (uint32_t)f2bf(a0) | ((uint32_t)f2bf(a1) << 16);
            }
        }
        __builtin_nontemporal_store((u32x4){pk[0], pk[1], pk[2], pk[3]}, (u32x4 *)(act + o));
        g = gn; u = un; q = qn;
    }
}

// The table is filled once per device, in stream order before its first reader, and the kernels that hold it in LDS get their
// dynamic LDS limit raised; callers on any host thread go through one lock. *ncu: the device's CU count.
static std::mutex g_lut_mu;
static struct { bool ready; int ncu; const uint16_t * lut; const uint16_t * small; } g_lut_dev[64];
static int silu_lut_ready(hipStream_t st, int * ncu, const uint16_t ** lut = nullptr, const uint16_t ** small = nullptr) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return CAMX_EINVAL;
    std::lock_guard<std::mutex> lock(g_lut_mu);
    if (!g_lut_dev[dev].ready) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return CAMX_EINVAL;
        silu_lut_fill<<<dim3(256), dim3(256), 0, st>>>();
        silu_small_fill<<<dim3((SWS_TAB + 255) / 256), dim3(256), 0, st>>>();
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
        if (hipFuncSetAttribute((const void *)swiglu_mmq_lut<MMQ_DS4, SRC_SWIGLU_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, SWM_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *)swiglu_mmq_lut<MMQ_D4, SRC_SWIGLU_BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, SWM_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *)silu_mul_lut, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) return CAMX_EINVAL;
        void * sym = nullptr, * sym_small = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_silu_lut)) != hipSuccess || !sym) return CAMX_EINVAL;
        if (hipGetSymbolAddress(&sym_small, HIP_SYMBOL(g_silu_small)) != hipSuccess || !sym_small) return CAMX_EINVAL;
        if (hipStreamSynchronize(st) != hipSuccess) return CAMX_EINVAL;     // later calls may come on other streams
        g_lut_dev[dev].lut = (const uint16_t *)sym;
        g_lut_dev[dev].small = (const uint16_t *)sym_small;
        g_lut_dev[dev].ncu = n;
        g_lut_dev[dev].ready = true;
    }
    *ncu = g_lut_dev[dev].ncu;
    if (lut) *lut = g_lut_dev[dev].lut;
    if (small) *small = g_lut_dev[dev].small;
    return CAMX_OK;
}
// the tables' device addresses for kernels of other files (filled and synchronized on first use)
__attribute__((visibility("hidden"))) int silu_lut_get(hipStream_t st, const uint16_t ** lut) {
    int ncu = 0;
    return silu_lut_ready(st, &ncu, lut);
}
__attribute__((visibility("hidden"))) int silu_luts_get(hipStream_t st, const uint16_t ** lut, const uint16_t ** small) {
    int ncu = 0;
    return silu_lut_ready(st, &ncu, lut, small);
}

// the wide form of silu_mul_bf16 (rows of H = 8 k values, 16-byte aligned, at least 2^22 values); CAMX_EINVAL: not applicable
__attribute__((visibility("hidden"))) int silu_mul_bf16_wide(const uint16_t * gu, uint16_t * act, int H, long n, hipStream_t st) {
    if (H % 8 || n < (1L << 22) || n / 8 >= 0x7fffffffL || (((uintptr_t)gu | (uintptr_t)act) & 15)) return CAMX_EINVAL;
    int ncu = 0;
    const int e = silu_lut_ready(st, &ncu);
    if (e) return e;
    silu_mul_lut<<<dim3((unsigned)ncu), dim3(1024), 131072, st>>>(gu, act, (unsigned)(H / 8), (unsigned)(n / 8));
    return (int)hipGetLastError();
}

extern "C" {

// gg_quantize_q8_1 (mode 0) and OP_GG_Q8_1's modes 1 / 2; y holds ceil(n / 32) blocks
int camx_gg_quantize_q8_1(const float * x, void * y, long n, int mode, float rs, const float * g, hipStream_t st) {
    if (n < 0 || !x || !y || mode < 0 || mode > 2 || (mode == 2 && !g) || ((uintptr_t)y & 3)) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    if (mode != 2 && n >= (1L << 20) && (((uintptr_t)x | (uintptr_t)y) & 15) == 0) {       // a batch that streams from HBM: one lane per block
        const long wgs = n / 8192;                                                           // whole workgroups of 4 x 2048 values
        if (wgs > 0x7fffffffL) return CAMX_EINVAL;
        if (mode == 0) q8_1_blocks<0><<<dim3((unsigned)wgs), dim3(256), 0, st>>>(x, (uint8_t *)y, rs);
        else q8_1_blocks<1><<<dim3((unsigned)wgs), dim3(256), 0, st>>>(x, (uint8_t *)y, rs);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess || n == wgs * 8192) return (int)e;
        x += wgs * 8192; y = (uint8_t *)y + wgs * (8192 / 32 * 36); n -= wgs * 8192;         // the rest: less than 8192 values
    }
    const long nstep = (n + 1023) >> 10;
    const int vec = ((uintptr_t)x & 15) == 0 && (mode != 2 || ((uintptr_t)g & 15) == 0);
    const int vecst = ((uintptr_t)y & 15) == 0;
    const long blocks = (nstep + 3) / 4;
    q8_1_flat<<<dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, st>>>(x, (uint8_t *)y, n, mode, rs, g, vec, vecst);
    CAMX_LAUNCH_RET();
}

// OP_GG_Q8_1 with its Seg fields in the tape's order (python/caminus/engine/k3.py:649-659): a = x, y, N = n, work = mode, rs = the SiLU
// pre-scale of mode 1, gs = the multiplier of mode 2
int camx_op_gg_q8_1(const float * x, void * y, int n, int work, float rs, const float * gs, hipStream_t st) {
    return camx_gg_quantize_q8_1(x, y, (long)n, work, rs, gs, st);
}

// quantize_mmq_q8_1<layout, false>: column c = row (ids ? ids[c] : c) of x (row stride s01 floats); ne00 = K, ne0 = K
// padded to 512, ne1 = ncols. The reference's s02 / s03 / ne2 (batch dims) must be 0 / 0 / 1.
int camx_quantize_mmq_q8_1(const float * x, const int32_t * ids, void * vy, long ne00, long s01, long s02, long s03,
                           long ne0, int ne1, int ne2, int n_expert_used, int layout, hipStream_t st) {
    (void)s02; (void)s03; (void)n_expert_used;
    if (!x || !vy || ne00 < 4 || ne00 % 4 || s01 < ne00 || s01 % 4 || ne0 % 512 || ne0 < ne00 || ne0 >= ne00 + 512 || ne1 < 0 || ne2 != 1 ||
        (layout != MMQ_D4 && layout != MMQ_DS4) || ((uintptr_t)x & 15) || ((uintptr_t)vy & 15)) return CAMX_EINVAL;
    if (ne1 >= 256 && (long)((ne1 + SWM_TOK - 1) / SWM_TOK) * (ne0 / 128) < 0x7ff00000L) {       // enough columns to fill the chip: persistent workgroups, block rows stored as whole aligned runs
        int dev = 0, ncu = 256;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return CAMX_EINVAL;
        const long ncol = ne0 / 128, nitems = (long)((ne1 + SWM_TOK - 1) / SWM_TOK) * ncol;
        if (ne1 >= 2048 && ncol <= 65535) {                                   // a prefill chunk: the one-shot form (no table for fp32 rows)
            launch_oneshot<SRC_F32>(x, ids, s01, ne00, vy, nullptr, ne1, ncol, layout, st);
            CAMX_LAUNCH_RET();
        }
        const long nwg = (nitems + 15) / 16;                                  // a small batch does not start workgroups that would only copy the table
        const dim3 grid((unsigned)(nwg < ncu ? nwg : ncu)), block(1024);
        if (layout == MMQ_DS4) swiglu_mmq_lut<MMQ_DS4, SRC_F32><<<grid, block, SWM_STAGE, st>>>(x, ids, s01, ne00, (uint8_t *)vy, nullptr, ne1, (unsigned)ncol, (unsigned)nitems);
        else swiglu_mmq_lut<MMQ_D4, SRC_F32><<<grid, block, SWM_STAGE, st>>>(x, ids, s01, ne00, (uint8_t *)vy, nullptr, ne1, (unsigned)ncol, (unsigned)nitems);
        CAMX_LAUNCH_RET();
    }
    MmqArgs a = {x, ids, (uint8_t *)vy, nullptr, ne00, ne0, s01, ne1, ne1, 0, nullptr};
    return launch_mmq<SRC_F32>(a, layout, st);
}

// quantize_mmq_q8_1<layout, true>: token t's row (stride s02 floats) quantized once and written to the columns
// ids[t * n_expert_used + slot] of the ne1 = ntok * n_expert_used compact columns
int camx_quantize_mmq_q8_1_scatter(const float * x, const int32_t * ids, void * vy, long ne00, long s01, long s02, long s03,
                                   long ne0, int ne1, int ne2, int n_expert_used, int layout, int ntok, hipStream_t st) {
    (void)s01; (void)s03;
    if (!x || !vy || !ids || ne00 < 4 || ne00 % 4 || s02 < ne00 || s02 % 4 || ne0 % 512 || ne0 < ne00 || ne0 >= ne00 + 512 || ne2 != 1 ||
        n_expert_used < 1 || ntok < 0 || ne1 != ntok * n_expert_used || (layout != MMQ_D4 && layout != MMQ_DS4) ||
        ((uintptr_t)x & 15) || ((uintptr_t)vy & 15)) return CAMX_EINVAL;
    if (ntok >= 2048 && ne0 / 128 <= 65535 && (long)ntok * n_expert_used < 0x7fffffffL) {      // a prefill chunk: the one-shot form
        launch_oneshot_scatter(x, ids, s02, ne00, vy, ntok, n_expert_used, ne1, ne0 / 128, layout, st);
        CAMX_LAUNCH_RET();
    }
    MmqArgs a = {x, ids, (uint8_t *)vy, nullptr, ne00, ne0, s02, ne1, ntok, n_expert_used, nullptr};
    return launch_mmq<SRC_F32>(a, layout, st);
}

// fused SwiGLU -> MMQ q8_1: gu bf16 [T][ld] = [g (F) | u (F)], act = bf16(bf16(silu g) * u) (kernels/core.hip:48-55) quantized
// as quantize_mmq_q8_1 of the fp32-widened act. act (optional) receives the bf16 activation [T][F].
int camx_swiglu_mmq_q8_1(const uint16_t * gu, long ld, long F, void * vy, uint16_t * act, int T, int layout, hipStream_t st) {
    if (!gu || !vy || F < 4 || F % 4 || ld < 2 * F || ld % 4 || T < 0 || (layout != MMQ_D4 && layout != MMQ_DS4) ||
        ((uintptr_t)gu & 7) || ((uintptr_t)vy & 15) || ((uintptr_t)act & 7)) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if (F % 8 == 0 && ld % 8 == 0 && !((uintptr_t)gu & 15) && !((uintptr_t)act & 15) &&
        (long)((T + SWM_TOK - 1) / SWM_TOK) * ((F + 511) / 512 * 4) < 0x7ff00000L) {
        int ncu = 0;
        const int rc = silu_lut_ready(st, &ncu);
        if (rc) return rc;
        const long Kp = (F + 511) / 512 * 512;
        const long ncol = Kp / 128, nitems = (long)((T + SWM_TOK - 1) / SWM_TOK) * ncol;
        const long nwg = (nitems + 15) / 16;                                  // a small batch does not start workgroups that would only copy the table
        const dim3 grid((unsigned)(nwg < ncu ? nwg : ncu)), block(1024);
        if (T >= 2048 && ncol <= 65535) {                                     // a prefill chunk: the one-shot form
            launch_oneshot<SRC_SWIGLU_BF16>(gu, nullptr, ld, F, vy, act, T, ncol, layout, st);
            CAMX_LAUNCH_RET();
        }
        if (layout == MMQ_DS4) swiglu_mmq_lut<MMQ_DS4, SRC_SWIGLU_BF16><<<grid, block, SWM_LDS, st>>>(gu, nullptr, ld, F, (uint8_t *)vy, act, T, (unsigned)ncol, (unsigned)nitems);
        else swiglu_mmq_lut<MMQ_D4, SRC_SWIGLU_BF16><<<grid, block, SWM_LDS, st>>>(gu, nullptr, ld, F, (uint8_t *)vy, act, T, (unsigned)ncol, (unsigned)nitems);
        CAMX_LAUNCH_RET();
    }
    const uint16_t * lut = nullptr;
    const int rc = silu_lut_get(st, &lut);
    if (rc) return rc;
    MmqArgs a = {gu, nullptr, (uint8_t *)vy, act, F, (F + 511) / 512 * 512, ld, T, T, 0, lut};
    return launch_mmq<SRC_SWIGLU_BF16>(a, layout, st);
}

}   // extern "C"
