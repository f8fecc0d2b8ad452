// Fused activation fake-quant (forward) for gfx950: per row of K values (K % 128 == 0, K <= 8192) a 128-point Hadamard
// rotation per chunk in bf16 steps, one int4-style scale per row, codes packed two per byte. Replaces actq_fwd_{f32,bf16},
// actq_fwd_codes_{f32,bf16}, silu_mul_actq_fwd and block_entry_fwd (kernels/actq.hip:40-53, 96-132, 247-274, 305-326).
//
// One 256-thread workgroup per row. A half-wave (32 lanes) transforms one 128-chunk: lane l holds elements 4l .. 4l + 3,
// butterfly stages 1-2 in registers, 4 .. 64 across lanes; a workgroup keeps 8 chunks in flight and up to 8 rounds of
// them in registers across the row-wide amax.
#include "common.cuh"

#define HSCALE 0.08837890625f      // bf16(1 / sqrt(128))
#define MAXR 8                     // rounds of 8 chunks: K <= 8 * 8 * 128

struct PlainF32 { const float * x; int K; CAMX_DEV f32x4 operator()(int row, int k) const { return *(const f32x4 *)(x + (size_t)row * K + k); } };
struct PlainBF16 { const uint16_t * x; int K; CAMX_DEV f32x4 operator()(int row, int k) const { return unpack_bf16x4(*(const u32x2 *)(x + (size_t)row * K + k)); } };
struct SiluMulSrc {
    const uint16_t * gu; int ld, F;
    CAMX_DEV f32x4 operator()(int row, int k) const {
        const uint16_t * r = gu + (size_t)row * ld;
        const f32x4 g = unpack_bf16x4(*(const u32x2 *)(r + k)), u = unpack_bf16x4(*(const u32x2 *)(r + F + k));
        f32x4 a;
        a.x = rbf(rbf(g.x / (1.0f + expf(-g.x))) * u.x); a.y = rbf(rbf(g.y / (1.0f + expf(-g.y))) * u.y);
        a.z = rbf(rbf(g.z / (1.0f + expf(-g.z))) * u.z); a.w = rbf(rbf(g.w / (1.0f + expf(-g.w))) * u.w);
        return a;
    }
};
struct RmsSrc {
    const float * x; const float * w; float rstd; int d;
    CAMX_DEV f32x4 operator()(int row, int k) const {
        const f32x4 xv = *(const f32x4 *)(x + (size_t)row * d + k), wv = *(const f32x4 *)(w + k);
        f32x4 a; a.x = xv.x * rstd * wv.x; a.y = xv.y * rstd * wv.y; a.z = xv.z * rstd * wv.z; a.w = xv.w * rstd * wv.w;
        return a;
    }
};

template <typename Src>
CAMX_DEV void actq_fwd_row(Src src, int row, uint16_t * __restrict__ y, float * __restrict__ s_out, int K, float clip, int qmax,
                           uint16_t * __restrict__ codes, float * lds) {
    const int tid = threadIdx.x, l = slot_of(tid) & 31, hw = tid >> 5, nch = K / 128;
    f32x4 u[MAXR];
    float amax = 0.0f;
#pragma unroll
    for (int c = 0; c < MAXR; c++) {
        const int ch = hw + 8 * c;
        const bool on = ch < nch;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (on) v = src(row, ch * 128 + 4 * l);
        v.x = rbf(v.x); v.y = rbf(v.y); v.z = rbf(v.z); v.w = rbf(v.w);        // autocast's bf16 input
        v = hadamard128_l4(v, l, false);
        v.x = rbf(v.x * HSCALE); v.y = rbf(v.y * HSCALE); v.z = rbf(v.z * HSCALE); v.w = rbf(v.w * HSCALE);
        u[c] = v;
        if (on) amax = fmaxf(amax, absmax4(v));
    }
    // row-wide max (order-free)
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    __syncthreads();
    if ((tid & 63) == 0) lds[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
    const float s = fmaxf(amax * clip / (float)qmax, 1e-8f);
    if (tid == 0 && s_out) s_out[row] = s;
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
#pragma unroll
    for (int c = 0; c < MAXR; c++) {
        const int ch = hw + 8 * c;
        if (ch < nch) {
            f32x4 q;
            q.x = fminf(fmaxf(rintf(u[c].x / s), lo), hi); q.y = fminf(fmaxf(rintf(u[c].y / s), lo), hi);
            q.z = fminf(fmaxf(rintf(u[c].z / s), lo), hi); q.w = fminf(fmaxf(rintf(u[c].w / s), lo), hi);
            if (y) { f32x4 d; d.x = q.x * s; d.y = q.y * s; d.z = q.z * s; d.w = q.w * s; *(u32x2 *)(y + (size_t)row * K + ch * 128 + 4 * l) = pack_f2bf_x4(d); }
            if (codes) {
                const uint32_t pk = ((uint32_t)(int)q.x & 0xfu) | (((uint32_t)(int)q.y & 0xfu) << 4) | (((uint32_t)(int)q.z & 0xfu) << 8) | (((uint32_t)(int)q.w & 0xfu) << 12);
                codes[(size_t)row * (K / 4) + ch * 32 + l] = (uint16_t)pk;
            }
        }
    }
}

template <typename Src>
__global__ void __launch_bounds__(256) actq_fwd_k(Src src, uint16_t * y, float * s, uint16_t * codes, int K, float clip, int qmax) {
    __shared__ float lds[4];
    actq_fwd_row(src, blockIdx.x, y, s, K, clip, qmax, codes, lds);
}

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

__global__ void __launch_bounds__(256) block_entry_fwd_k(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y,
                                                         float * s, uint16_t * codes, uint16_t * ab, float * rstd_out, int d, float clip, int qmax) {
    __shared__ float lds[4];
    __shared__ float slot;
    const int row = blockIdx.x;
    const float * xr = x + (size_t)row * d;
    const float ss = row_tree_sum(SqTerm{xr}, d, &slot);
    const float rstd = rsqrt_exact(ss / (float)d + eps);
    if (threadIdx.x == 0 && rstd_out) rstd_out[row] = rstd;
    actq_fwd_row(RmsSrc{x, nw, rstd, d}, row, y, s, d, clip, qmax, codes, lds);
    for (int j = 0; j < nab; j++) {
        const float v = row_tree_sum(AbTerm{xr, nw, rstd, wab + (size_t)j * d}, d, &slot);
        if (threadIdx.x == 0) ab[(size_t)row * nab + j] = f2bf(v);
    }
}

static int actq_check(int K, int qmax, int M) { return (K < 128 || K % 128 || K > 8192 || qmax < 1 || M < 0) ? CAMX_EINVAL : CAMX_OK; }

extern "C" {

// actq_fwd_{f32,bf16} and actq_fwd_codes_{f32,bf16}: y bf16 [M][K] (optional when codes are written), s [M] (optional),
// codes [M][K / 2] bytes (optional; needs qmax <= 7)
int camx_actq_fwd(const void * x, int is_bf16, uint16_t * y, float * s, uint16_t * codes, int K, float clip, int qmax, int M, hipStream_t st) {
    if (!x || (!y && !codes) || actq_check(K, qmax, M) || ((uintptr_t)x & (is_bf16 ? 7 : 15)) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    if (is_bf16) actq_fwd_k<<<dim3(M), dim3(256), 0, st>>>(PlainBF16{(const uint16_t *)x, K}, y, s, codes, K, clip, qmax);
    else actq_fwd_k<<<dim3(M), dim3(256), 0, st>>>(PlainF32{(const float *)x, K}, y, s, codes, K, clip, qmax);
    CAMX_LAUNCH_RET();
}
int camx_silu_mul_actq_fwd(const uint16_t * gu, int ld, int F, uint16_t * y, float * s, uint16_t * codes, float clip, int qmax, int M, hipStream_t st) {
    if (!gu || (!y && !codes) || actq_check(F, qmax, M) || ld < 2 * F || (ld & 3) || ((uintptr_t)gu & 7) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    actq_fwd_k<<<dim3(M), dim3(256), 0, st>>>(SiluMulSrc{gu, ld, F}, y, s, codes, F, clip, qmax);
    CAMX_LAUNCH_RET();
}
int camx_block_entry_fwd(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y, float * s, uint16_t * codes,
                         uint16_t * ab, float * rstd_out, int d, float clip, int qmax, int M, hipStream_t st) {
    if (!x || !nw || (!y && !codes) || actq_check(d, qmax, M) || nab < 0 || nab > 16 || (nab && (!wab || !ab)) || ((uintptr_t)x & 15) ||
        ((uintptr_t)nw & 15) || ((uintptr_t)wab & 7) || ((uintptr_t)y & 7) || ((uintptr_t)codes & 1)) return CAMX_EINVAL;
    if (M == 0) return CAMX_OK;
    block_entry_fwd_k<<<dim3(M), dim3(256), 0, st>>>(x, nw, wab, nab, eps, y, s, codes, ab, rstd_out, d, clip, qmax);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
