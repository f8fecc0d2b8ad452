// Activation quantizers for gfx950: ggml q8_1 blocks (36 B / 32 values) and the MMQ layout (144 B / 128 values), plain,
// behind SwiGLU, and scattered to expert columns. Replaces gg_quantize_q8_1 / OP_GG_Q8_1 (kernels/k3_gguf.hip:29-36,
// kernels/k3_gguf_ops.h:55-77,146-162) and quantize_mmq_q8_1<layout, scatter> (kernels/ggml_mmq/quantize_mmq.cuh:41-140).
//
// Layout: 8 lanes x 4 consecutive floats = one 32-value quantization group; a wave covers 256 values per step with one
// 128-bit load per lane and writes each group's 32 codes as 8 dwords.
#include "common.cuh"

CAMX_DEV float silu_f(float x) { return x / (1.0f + expf(-x)); }

// ---- q8_1, flat -------------------------------------------------------------------------------------------------------------
// mode 0 plain, 1 silu(x * rs), 2 silu(x) * g[i]; values past n quantize as 0; blocks = ceil(n / 32)
__global__ void __launch_bounds__(256) q8_1_flat(const float * __restrict__ x, uint8_t * __restrict__ y, long n, int mode, float rs,
                                                 const float * __restrict__ g, int vec) {
    const int lane = threadIdx.x & 63;
    const long wave = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long nwaves = (long)gridDim.x * 4;
    const long nslab = (n + 255) >> 8, nb = (n + 31) >> 5;
    for (long s = wave; s < nslab; s += nwaves) {
        const long i0 = s * 256 + 4 * lane;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f}, gv = {0.0f, 0.0f, 0.0f, 0.0f};
        if (vec && i0 + 3 < n) {
            v = *(const f32x4 *)(x + i0);
            if (mode == 2) gv = *(const f32x4 *)(g + i0);
        } else {
            float t[4] = {0.0f, 0.0f, 0.0f, 0.0f}, tg[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int k = 0; k < 4; k++) if (i0 + k < n) { t[k] = x[i0 + k]; if (mode == 2) tg[k] = g[i0 + k]; }
            v = (f32x4){t[0], t[1], t[2], t[3]}; gv = (f32x4){tg[0], tg[1], tg[2], tg[3]};
        }
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
        const long b = s * 8 + (lane >> 3);
        if (b < nb) q8_1_emit(v, y + b * 36, lane & 7);     // (a group of 8 lanes is wholly inside or outside)
    }
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
};

CAMX_DEV f32x4 swiglu_bf16x4(u32x2 gw, u32x2 uw, u32x2 * packed) {
    const f32x4 g = unpack_bf16x4(gw), u = unpack_bf16x4(uw);
    f32x4 a;
    a.x = rbf(g.x / (1.0f + expf(-g.x))) * u.x; a.y = rbf(g.y / (1.0f + expf(-g.y))) * u.y;
    a.z = rbf(g.z / (1.0f + expf(-g.z))) * u.z; a.w = rbf(g.w / (1.0f + expf(-g.w))) * u.w;
    const u32x2 p = pack_f2bf_x4(a);
    *packed = p;
    return unpack_bf16x4(p);
}

template <int LAYOUT, int SRC>
__global__ void __launch_bounds__(256) mmq_q8_1_rows(MmqArgs a) {
    const int lane = threadIdx.x & 63;
    const int col = blockIdx.x * 4 + (threadIdx.x >> 6);            // source row index
    if (col >= a.nsrc) return;
    const long slab = blockIdx.y;                                   // 256 values = 2 blocks of 128
    const long i0 = slab * 256 + 4 * lane;
    if (i0 >= a.Kp) return;                                         // (Kp is a multiple of 512: never taken for half a wave)
    const long srow = a.kexp ? col : (a.ids ? a.ids[col] : col);
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i0 < a.K) {                                                 // K % 4 == 0: a lane's four values are in or out together
        if (SRC == SRC_F32) v = *(const f32x4 *)((const float *)a.x + srow * a.stride + i0);
        else {
            const uint16_t * r = (const uint16_t *)a.x + srow * a.stride;
            u32x2 packed;
            v = swiglu_bf16x4(*(const u32x2 *)(r + i0), *(const u32x2 *)(r + a.K + i0), &packed);
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
        const long dcol = a.kexp ? a.ids[(long)col * a.kexp + slot] : col;
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

extern "C" {

// gg_quantize_q8_1 (mode 0) and OP_GG_Q8_1's modes 1 / 2; y holds ceil(n / 32) blocks
int camx_gg_quantize_q8_1(const float * x, void * y, long n, int mode, float rs, const float * g, hipStream_t st) {
    if (n < 0 || !x || !y || mode < 0 || mode > 2 || (mode == 2 && !g) || ((uintptr_t)y & 3)) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const long nslab = (n + 255) >> 8;
    const int vec = ((uintptr_t)x & 15) == 0 && (mode != 2 || ((uintptr_t)g & 15) == 0);
    const long blocks = (nslab + 3) / 4;
    q8_1_flat<<<dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, st>>>(x, (uint8_t *)y, n, mode, rs, g, vec);
    CAMX_LAUNCH_RET();
}

// quantize_mmq_q8_1<layout, false>: column c = row (ids ? ids[c] : c) of x (row stride s01 floats); ne00 = K, ne0 = K
// padded to 512, ne1 = ncols. The reference's s02 / s03 / ne2 (batch dims) must be 0 / 0 / 1.
int camx_quantize_mmq_q8_1(const float * x, const int32_t * ids, void * vy, long ne00, long s01, long s02, long s03,
                           long ne0, int ne1, int ne2, int n_expert_used, int layout, hipStream_t st) {
    (void)s02; (void)s03; (void)n_expert_used;
    if (!x || !vy || ne00 < 4 || ne00 % 4 || s01 < ne00 || s01 % 4 || ne0 % 512 || ne0 < ne00 || ne0 >= ne00 + 512 || ne1 < 0 || ne2 != 1 ||
        (layout != MMQ_D4 && layout != MMQ_DS4) || ((uintptr_t)x & 15) || ((uintptr_t)vy & 15)) return CAMX_EINVAL;
    MmqArgs a = {x, ids, (uint8_t *)vy, nullptr, ne00, ne0, s01, ne1, ne1, 0};
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
    MmqArgs a = {x, ids, (uint8_t *)vy, nullptr, ne00, ne0, s02, ne1, ntok, n_expert_used};
    return launch_mmq<SRC_F32>(a, layout, st);
}

// fused SwiGLU -> MMQ q8_1: gu bf16 [T][ld] = [g (F) | u (F)], act = bf16(bf16(silu g) * u) (kernels/core.hip:48-55) quantized
// as quantize_mmq_q8_1 of the fp32-widened act. act (optional) receives the bf16 activation [T][F].
int camx_swiglu_mmq_q8_1(const uint16_t * gu, long ld, long F, void * vy, uint16_t * act, int T, int layout, hipStream_t st) {
    if (!gu || !vy || F < 4 || F % 4 || ld < 2 * F || ld % 4 || T < 0 || (layout != MMQ_D4 && layout != MMQ_DS4) ||
        ((uintptr_t)gu & 7) || ((uintptr_t)vy & 15) || ((uintptr_t)act & 7)) return CAMX_EINVAL;
    MmqArgs a = {gu, nullptr, (uint8_t *)vy, act, F, (F + 511) / 512 * 512, ld, T, T, 0};
    return launch_mmq<SRC_SWIGLU_BF16>(a, layout, st);
}

}   // extern "C"
