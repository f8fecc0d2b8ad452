// Elementwise and small row kernels for gfx950: SwiGLU and sigmoid gates, the GDN short convolution and L2 norm, and the
// S1 core's gather / cast / residual kernels. Replaces q3p_swiglu / OP_OWN_SWIGLU16 (kernels/q3m_prefill.hip:516-518,
// kernels/k3_own_ops.h:258-262), gg_silu_mul (kernels/k3_gguf.hip:74-77), pf_gate_mul / q35p_gate_mul16
// (kernels/prefill_attn.hip:379-386, kernels/q35_prefill.hip:960-969), pf_gdn_conv / pf_conv_state
// (kernels/prefill_glue.hip:314-341), pf_gdn_l2 (kernels/prefill_gdn.hip:66-78), kernels/core.hip and
// residual_slices_fwd (kernels/fuse.hip:19-33). Four elements per lane, 128-bit accesses where alignment allows.
#include "common.cuh"

CAMX_DEV float silu_f(float x) { return x / (1.0f + expf(-x)); }
CAMX_DEV float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
// for results that are rounded to 16 bits right away (tolerance: one unit of the 16-bit format): v_exp_f32 and v_rcp_f32, each
// good to about 1e-6 relative, in place of the library exponential and the IEEE division (6 instructions instead of 30: the
// 16-bit elementwise kernels are otherwise bound by the vector ALU, not by HBM). exp overflow gives 1 / inf = 0, as the division does.
CAMX_DEV float sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
CAMX_DEV float silu_fast(float x) { return x * sigmoid_fast(x); }

#define GRID_1D(n4) dim3((unsigned)((((n4) + 255) / 256) < 1048576 ? (((n4) + 255) / 256) : 1048576))

// y16[i] = fp16(silu(g[i]) * u[i]); out_f32: y32[i] = silu(g[i]) * u[i]
template <bool F16OUT>
__global__ void __launch_bounds__(256) swiglu_f32(const float * __restrict__ g, const float * __restrict__ u, void * __restrict__ y, long n, int vec) {
    const long stride = (long)gridDim.x * 256;
    for (long q = (long)blockIdx.x * 256 + threadIdx.x; q * 4 < n; q += stride) {
        const long i = q * 4;
        float gv[4], uv[4], r[4];
        if (vec && i + 3 < n) {
            const f32x4 a = __builtin_nontemporal_load((const f32x4 *)(g + i)), b = __builtin_nontemporal_load((const f32x4 *)(u + i));
            gv[0] = a.x; gv[1] = a.y; gv[2] = a.z; gv[3] = a.w; uv[0] = b.x; uv[1] = b.y; uv[2] = b.z; uv[3] = b.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++) { gv[k] = i + k < n ? g[i + k] : 0.0f; uv[k] = i + k < n ? u[i + k] : 0.0f; }
        }
#pragma unroll
        for (int k = 0; k < 4; k++) r[k] = gv[k] / (1.0f + expf(-gv[k])) * uv[k];
        if (vec && i + 3 < n) {
            if (F16OUT) __builtin_nontemporal_store(pack_f16x4((f32x4){r[0], r[1], r[2], r[3]}), (u32x2 *)((uint16_t *)y + i));
            else __builtin_nontemporal_store((f32x4){r[0], r[1], r[2], r[3]}, (f32x4 *)((float *)y + i));
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (i + k < n) { if (F16OUT) ((uint16_t *)y)[i + k] = f2h_bits(r[k]); else ((float *)y)[i + k] = r[k]; }
        }
    }
}

// silu_mul_bf16: act[r][c] = bf16(bf16(silu(g)) * u), gu rows = [g (H) | u (H)]
// bf16(silu g) comes from the 65536-entry table in device memory (the one the wide form and the SwiGLU -> MMQ kernel hold in
// LDS), so a row's result does not depend on which of them a batch size selects
__global__ void __launch_bounds__(256) silu_mul_bf16_k(const uint16_t * __restrict__ gu, uint16_t * __restrict__ act, int H, long n, int vec,
                                                       const uint16_t * __restrict__ lut) {
    const long stride = (long)gridDim.x * 256;
    for (long q = (long)blockIdx.x * 256 + threadIdx.x; q * 4 < n; q += stride) {
        const long i = q * 4;
        if (vec) {     // H % 4 == 0: the four elements share a row
            const long r = i / H, c = i - r * H;
            const u32x2 gw = *(const u32x2 *)(gu + r * 2 * H + c);
            const f32x4 u = unpack_bf16x4(*(const u32x2 *)(gu + r * 2 * H + H + c));
            f32x4 a;
            a.x = bf2f(lut[gw.x & 0xffffu]) * u.x; a.y = bf2f(lut[gw.x >> 16]) * u.y; a.z = bf2f(lut[gw.y & 0xffffu]) * u.z; a.w = bf2f(lut[gw.y >> 16]) * u.w;
            *(u32x2 *)(act + i) = pack_f2bf_x4(a);
        } else {
            for (int k = 0; k < 4 && i + k < n; k++) {
                const long r = (i + k) / H, c = (i + k) - r * H;
                const float u = bf2f(gu[r * 2 * H + H + c]);
                act[i + k] = f2bf(bf2f(lut[gu[r * 2 * H + c]]) * u);
            }
        }
    }
}

// y[i] = a[i] * sigmoid(gate[(i / D) * stride + off + i % D]); IO 0: fp32 a, gate -> fp32 y; 1: fp32 -> fp16 y;
// 2: bf16 a, gate -> bf16 y (to_bf16)
template <int IO>
__global__ void __launch_bounds__(256) gate_mul_k(const void * __restrict__ a, const void * __restrict__ gt, void * __restrict__ y, long N, int D,
                                                  int stride, int off) {
    const long step = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < N; i += step) {
        const long h = i / D; const int d = (int)(i - h * D);
        const size_t gi = (size_t)h * stride + off + d;
        const float gv = IO == 2 ? bf2f(((const uint16_t *)gt)[gi]) : ((const float *)gt)[gi];
        const float av = IO == 2 ? bf2f(((const uint16_t *)a)[i]) : ((const float *)a)[i];
        const float sgm = 1.0f / (1.0f + expf(-gv));
        const float v = av * sgm;
        if (IO == 0) ((float *)y)[i] = v; else if (IO == 1) ((uint16_t *)y)[i] = f2h_bits(v); else ((uint16_t *)y)[i] = to_bf16(v);
    }
}

// the same, VW consecutive values per thread with 128-bit accesses (VW = 4 for fp32 inputs, 8 for bf16): D, stride, off
// multiples of VW and 16-byte aligned bases, so a vector never straddles a head
template <int IO>
__global__ void __launch_bounds__(256) gate_mul_vec(const void * __restrict__ a, const void * __restrict__ gt, void * __restrict__ y, long nvec, int dv,
                                                    int stride, int off) {
    constexpr int VW = IO == 2 ? 8 : 4;
    const long step = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += step) {
        const long h = i / dv; const int d = (int)(i - h * dv) * VW;
        const size_t gi = (size_t)h * stride + off + d, ai = (size_t)i * VW;
        float av[VW], gv[VW], v[VW];
        if (IO == 2) {
            const u32x4 aw = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)a + ai)), gw = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)gt + gi));
#pragma unroll
            for (int p = 0; p < 4; p++) {
                av[2 * p] = __builtin_bit_cast(float, aw[p] << 16); av[2 * p + 1] = __builtin_bit_cast(float, aw[p] & 0xffff0000u);
                gv[2 * p] = __builtin_bit_cast(float, gw[p] << 16); gv[2 * p + 1] = __builtin_bit_cast(float, gw[p] & 0xffff0000u);
            }
        } else {
            const f32x4 aw = __builtin_nontemporal_load((const f32x4 *)((const float *)a + ai)), gw = __builtin_nontemporal_load((const f32x4 *)((const float *)gt + gi));
#pragma unroll
            for (int k = 0; k < 4; k++) { av[k] = aw[k]; gv[k] = gw[k]; }
        }
#pragma unroll
        for (int k = 0; k < VW; k++) { const float sgm = IO == 0 ? 1.0f / (1.0f + expf(-gv[k])) : sigmoid_fast(gv[k]); v[k] = av[k] * sgm; }
        if (IO == 0) __builtin_nontemporal_store((f32x4){v[0], v[1], v[2], v[3]}, (f32x4 *)((float *)y + ai));
        else if (IO == 1) __builtin_nontemporal_store(pack_f16x4((f32x4){v[0], v[1], v[2], v[3]}), (u32x2 *)((uint16_t *)y + ai));
        else {
            const u32x2 lo = pack_bf16x4_rne((f32x4){v[0], v[1], v[2], v[3]}), hi = pack_bf16x4_rne((f32x4){v[4 % VW], v[5 % VW], v[6 % VW], v[7 % VW]});
            __builtin_nontemporal_store((u32x4){lo.x, lo.y, hi.x, hi.y}, (u32x4 *)((uint16_t *)y + ai));
        }
    }
}

// y[t, c] = silu(fma chain over [x(t-3), x(t-2), x(t-1), x(t)] . w[c]), negative times from st[c] = [x(-3), x(-2), x(-1)]
template <bool BF16>
__global__ void __launch_bounds__(256) gdn_conv_k(const void * __restrict__ x, const float * __restrict__ w, const float * __restrict__ st,
                                                  void * __restrict__ y, int C, int T, int ldx, int ldy) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)T * C) return;
    const int t = (int)(i / C), c = (int)(i - (long)t * C);
    const f32x4 w4 = *(const f32x4 *)(w + (size_t)c * 4);
    float in[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int tj = t - 3 + j;
        if (tj >= 0) in[j] = BF16 ? bf2f(((const uint16_t *)x)[(size_t)tj * ldx + c]) : ((const float *)x)[(size_t)tj * ldx + c];
        else in[j] = st[(size_t)c * 3 + 3 + tj];
    }
    float sumf = 0.0f;
    sumf = __builtin_fmaf(in[0], w4.x, sumf); sumf = __builtin_fmaf(in[1], w4.y, sumf);
    sumf = __builtin_fmaf(in[2], w4.z, sumf); sumf = __builtin_fmaf(in[3], w4.w, sumf);
    const float r = BF16 ? silu_fast(sumf) : silu_f(sumf);           // bf16 rows: the streaming kernel's form, so a token's bits do not depend on the chunk it came in
    if (BF16) ((uint16_t *)y)[(size_t)t * ldy + c] = to_bf16(r); else ((float *)y)[(size_t)t * ldy + c] = r;
}
// OP_GDN_CONV (kernels/k3_q35_ops.h:148-177): the decode / verify form with a lazy commit. Per channel: the state [3] first takes in
// the mprev tokens of the previous pass that were accepted (its inputs, kept in xprev), and is stored; then the T tokens of this
// pass are convolved from that state without committing them, and become the next pass's xprev. One thread per channel, the
// window in registers; the same fma chain and silu as the kernel above.
__global__ void __launch_bounds__(256) op_gdn_conv_k(const float * __restrict__ w, float * __restrict__ st, const float * __restrict__ x,
                                                     const int32_t * __restrict__ params, float * __restrict__ y, float * __restrict__ xprev, int C, int T) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    int mprev = params[1];
    mprev = mprev < 0 ? 0 : (mprev > T ? T : mprev);                 // (the host refuses a commit outside [0, T]; never read past xprev's rows)
    float s0 = st[(size_t)c * 3], s1 = st[(size_t)c * 3 + 1], s2 = st[(size_t)c * 3 + 2];
    const f32x4 w4 = *(const f32x4 *)(w + (size_t)c * 4);
    for (int j = 0; j < mprev; j++) { s0 = s1; s1 = s2; s2 = xprev[(size_t)j * C + c]; }
    st[(size_t)c * 3] = s0; st[(size_t)c * 3 + 1] = s1; st[(size_t)c * 3 + 2] = s2;
    for (int t0 = 0; t0 < T; t0 += 8) {                              // eight tokens' inputs requested together: a pass is latency, not bytes
        float xv[8];
#pragma unroll
        for (int u = 0; u < 8; u++) xv[u] = x[(size_t)(t0 + u < T ? t0 + u : T - 1) * C + c];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int t = t0 + u;
            if (t >= T) break;
            float sumf = 0.0f;
            sumf = __builtin_fmaf(s0, w4.x, sumf); sumf = __builtin_fmaf(s1, w4.y, sumf);
            sumf = __builtin_fmaf(s2, w4.z, sumf); sumf = __builtin_fmaf(xv[u], w4.w, sumf);
            y[(size_t)t * C + c] = silu_f(sumf);
            s0 = s1; s1 = s2; s2 = xv[u];
            xprev[(size_t)t * C + c] = xv[u];
        }
    }
}
// Prefill chunks: a lane owns VW consecutive channels and walks TR consecutive tokens, with the rows of the next eight tokens
// always in flight (a ring of eight 128-bit loads that is refilled as it is consumed) and the four-tap window in registers;
// one wave per workgroup, so the grid's (channel groups x token ranges) waves spread evenly over the chip.
// L2: the L2 norm of the q / k heads (the first heads * 128 channels) in the same pass, from the values as they are stored: qk
// [T][heads][128]. A head is 16 lanes x 8 channels (bf16 rows) or 32 lanes x 4 (fp32 rows, the lanes in slot order), whole heads per
// wave (C % 128 == 0), so every lane of a head is present.
CAMX_DEV void l2_head_w8(const float (&v)[8], float (&o)[8], float rs);
CAMX_DEV f32x4 l2_head_l4(f32x4 v, int lane, float rs);
template <bool BF16, bool L2 = false>
__global__ void __launch_bounds__(64) gdn_conv_stream(const void * __restrict__ x, const float * __restrict__ w, const float * __restrict__ st,
                                                      void * __restrict__ y, int C, int T, int ldx, int ldy, int TR,
                                                      void * __restrict__ qk = nullptr, int heads = 0, float rs = 0.0f) {
    constexpr int VW = BF16 ? 8 : 4, P = 8;
    const int lane_l2 = slot_of(threadIdx.x);
    const int cv = blockIdx.x * 64 + (L2 && !BF16 ? lane_l2 : (int)threadIdx.x);
    if (cv * VW >= C) return;
    const int c0 = cv * VW, t0 = blockIdx.y * TR, t1 = T < t0 + TR ? T : t0 + TR;
    auto row = [&](int t) {                                            // (a row index past the batch is clamped: the load is harmless and never used)
        const int tc = t < T - 1 ? t : T - 1;
        return BF16 ? __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)x + (size_t)tc * ldx + c0))
                    : __builtin_nontemporal_load((const u32x4 *)((const float *)x + (size_t)tc * ldx + c0));
    };
    auto widen = [&](float (&o)[VW], u32x4 r) {
        if (BF16) {
#pragma unroll
            for (int p = 0; p < 4; p++) { const uint32_t b = r[p]; o[2 * p] = __builtin_bit_cast(float, b << 16); o[(2 * p + 1) % VW] = __builtin_bit_cast(float, b & 0xffff0000u); }
        } else {
#pragma unroll
            for (int p = 0; p < 4; p++) { const uint32_t b = r[p]; o[p % VW] = __builtin_bit_cast(float, b); }
        }
    };
    u32x4 halo[3];                                                     // the three rows before the range (another wave's tokens; clamped when the state stands in)
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int tj = t0 - 3 + j < 0 ? 0 : t0 - 3 + j;
        halo[j] = BF16 ? *(const u32x4 *)((const uint16_t *)x + (size_t)tj * ldx + c0) : *(const u32x4 *)((const float *)x + (size_t)tj * ldx + c0);
    }
    u32x4 ring[P];
#pragma unroll
    for (int u = 0; u < P; u++) ring[u] = row(t0 + u);
    f32x4 w4[VW];
#pragma unroll
    for (int k = 0; k < VW; k++) w4[k] = *(const f32x4 *)(w + (size_t)(c0 + k) * 4);
    float win[4][VW];                                                  // token t0 - 3 + j sits in slot j & 3
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int tj = t0 - 3 + j;
        if (tj < 0) {
#pragma unroll
            for (int k = 0; k < VW; k++) win[j][k] = st[(size_t)(c0 + k) * 3 + 3 + tj];
        } else widen(win[j], halo[j]);
    }
    auto emit = [&](int tt, int u) {                                   // token tt's output from window slots u .. u + 3 (mod 4)
        float r[VW];
#pragma unroll
        for (int k = 0; k < VW; k++) {
            float sumf = 0.0f;
            sumf = __builtin_fmaf(win[u & 3][k], w4[k].x, sumf); sumf = __builtin_fmaf(win[(u + 1) & 3][k], w4[k].y, sumf);
            sumf = __builtin_fmaf(win[(u + 2) & 3][k], w4[k].z, sumf); sumf = __builtin_fmaf(win[(u + 3) & 3][k], w4[k].w, sumf);
            r[k] = BF16 ? silu_fast(sumf) : silu_f(sumf);
        }
        const size_t o = (size_t)tt * ldy + c0;
        if (BF16) {
            const u32x2 lo = pack_bf16x4_rne((f32x4){r[0], r[1], r[2], r[3]}), hi = pack_bf16x4_rne((f32x4){r[4 % VW], r[5 % VW], r[6 % VW], r[7 % VW]});
            if (!L2 || y) __builtin_nontemporal_store((u32x4){lo.x, lo.y, hi.x, hi.y}, (u32x4 *)((uint16_t *)y + o));     // (on cold lines: 38.5 us against 42.2 with plain stores, 4096 x 10240)
            if constexpr (L2) {
                const f32x4 a = unpack_bf16x4(lo), b = unpack_bf16x4(hi);
                const float v8[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                float o8[8];
                l2_head_w8(v8, o8, rs);
                if (c0 < heads * 128) {
                    const u32x2 pa = pack_bf16x4_rne((f32x4){o8[0], o8[1], o8[2], o8[3]}), pb = pack_bf16x4_rne((f32x4){o8[4], o8[5], o8[6], o8[7]});
                    __builtin_nontemporal_store((u32x4){pa.x, pa.y, pb.x, pb.y}, (u32x4 *)((uint16_t *)qk + (size_t)tt * heads * 128 + c0));
                }
            }
        } else {
            if (!L2 || y) __builtin_nontemporal_store((f32x4){r[0], r[1], r[2], r[3]}, (f32x4 *)((float *)y + o));
            if constexpr (L2) {
                const f32x4 q4 = l2_head_l4((f32x4){r[0], r[1], r[2], r[3]}, lane_l2, rs);
                if (c0 < heads * 128) __builtin_nontemporal_store(q4, (f32x4 *)((float *)qk + (size_t)tt * heads * 128 + c0));
            }
        }
    };
    int t = t0;
    // No row past the wave's range is requested: it is another wave's, and would come from HBM twice (with eight rows requested ahead
    // regardless, 4096 x 10240 read 34 % more than its input, 16384 tokens 17 %). The last group asks for the range's last row again
    // instead, which is still on its way or in L2 (+ 3 % of reads); a branch around the request would do without that, but with it the
    // compiler keeps all eight tokens of a group live at once (fp32 rows: 404 registers instead of 92).
    for (; t + P <= t1; t += P) {                                      // whole groups of eight tokens
#pragma unroll
        for (int u = 0; u < P; u++) {
            // the whole row is widened before its ring slot is requested again: left to itself the compiler widens half of it later,
            // keeps that half in a copy, and hoists the copies of all eight slots (and the waits for their loads) to the top of the loop
            widen(win[(u + 3) & 3], ring[u]);
            if constexpr (BF16) {
#pragma unroll
                for (int k = 0; k < VW; k++) asm volatile("" : "+v"(win[(u + 3) & 3][k]));
                __builtin_amdgcn_sched_barrier(0);
            }
            ring[u] = row(t + u + P < t1 ? t + u + P : t1 - 1);
            if constexpr (BF16) __builtin_amdgcn_sched_barrier(0);
            emit(t + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < P; u++)                                        // the last, partial group
        if (t + u < t1) { widen(win[(u + 3) & 3], ring[u]); emit(t + u, u); __builtin_amdgcn_sched_barrier(0); }
}

template <bool BF16>
__global__ void __launch_bounds__(256) conv_state_k(const void * __restrict__ x, float * __restrict__ st, int C, int T, int ldx) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float s[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int tj = T - 3 + j;
        if (tj >= 0) s[j] = BF16 ? bf2f(((const uint16_t *)x)[(size_t)tj * ldx + c]) : ((const float *)x)[(size_t)tj * ldx + c];
        else s[j] = st[(size_t)c * 3 + 3 + tj];
    }
#pragma unroll
    for (int j = 0; j < 3; j++) st[(size_t)c * 3 + j] = s[j];
}

// per head of K <= 512 values: y = (scale * x) * (1 / sqrt(K)), scale = 1 / sqrt(sum x^2 / K + rs); one wave per head
template <bool BF16, bool VEC>
__global__ void __launch_bounds__(256) gdn_l2_k(const void * __restrict__ x, void * __restrict__ y, int heads, int K, int ldx, float rs, int total) {
    const int lane = slot_of(threadIdx.x & 63);
    const int t = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (t >= total) return;
    const int tt = t / heads, hh = t - tt * heads;
    const size_t xo = (size_t)tt * ldx + (size_t)hh * K, yo = (size_t)t * K;
    float xv[2][4];
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int i0 = 256 * j + 4 * lane;
        if (VEC) {                                          // K, ldx multiples of 4 and aligned bases: four values in or out together
            f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (i0 < K) v = BF16 ? unpack_bf16x4(*(const u32x2 *)((const uint16_t *)x + xo + i0)) : *(const f32x4 *)((const float *)x + xo + i0);
            xv[j][0] = v.x; xv[j][1] = v.y; xv[j][2] = v.z; xv[j][3] = v.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = i0 + k;
                xv[j][k] = 0.0f;
                if (i < K) xv[j][k] = BF16 ? bf2f(((const uint16_t *)x)[xo + i]) : ((const float *)x)[xo + i];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {   // (an absent element adds fma(0, 0, s) = s: the tree's threads past K hold 0)
        ss.x = __builtin_fmaf(xv[j][0], xv[j][0], ss.x); ss.y = __builtin_fmaf(xv[j][1], xv[j][1], ss.y);
        ss.z = __builtin_fmaf(xv[j][2], xv[j][2], ss.z); ss.w = __builtin_fmaf(xv[j][3], xv[j][3], ss.w);
    }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)K + rs), s2 = 1.0f / sqrtf((float)K);
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int i0 = 256 * j + 4 * lane;
        f32x4 v;
        v.x = (scale * xv[j][0]) * s2; v.y = (scale * xv[j][1]) * s2; v.z = (scale * xv[j][2]) * s2; v.w = (scale * xv[j][3]) * s2;
        if (VEC) {
            if (i0 < K) { if (BF16) *(u32x2 *)((uint16_t *)y + yo + i0) = pack_bf16x4_rne(v); else *(f32x4 *)((float *)y + yo + i0) = v; }
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (i0 + k < K) { if (BF16) ((uint16_t *)y)[yo + i0 + k] = to_bf16(v[k]); else ((float *)y)[yo + i0 + k] = v[k]; }
        }
    }
}

// K = 128 (the GDN key heads): a half-wave per head, two heads per wave, 128-bit accesses, U heads per half-wave with all
// their loads issued first (a head is only 256 - 512 bytes). The logical threads past 128 hold zeros in the reference's
// tree, so the four group sums of the head added in order are the whole sum.
template <bool BF16, int U>
__global__ void __launch_bounds__(256) gdn_l2_128(const void * __restrict__ x, void * __restrict__ y, int heads, int ldx, float rs, int total) {
    const int lane = slot_of(threadIdx.x & 63), l = lane & 31;
    const int span = gridDim.x * 8;                                  // heads per pass of the grid
    const int t0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = t0 + u * span, tc = t < total ? t : 0;
        const int tt = tc / heads, hh = tc - tt * heads;
        const size_t xo = (size_t)tt * ldx + (size_t)hh * 128 + 4 * l;
        v[u] = BF16 ? unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)((const uint16_t *)x + xo)))
                    : __builtin_nontemporal_load((const f32x4 *)((const float *)x + xo));
    }
    const float s2 = 1.0f / sqrtf(128.0f);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = t0 + u * span;
        f32x4 ss;
        ss.x = __builtin_fmaf(v[u].x, v[u].x, 0.0f); ss.y = __builtin_fmaf(v[u].y, v[u].y, 0.0f);
        ss.z = __builtin_fmaf(v[u].z, v[u].z, 0.0f); ss.w = __builtin_fmaf(v[u].w, v[u].w, 0.0f);
        const float tot = half_groups_in_order<4>(group32_sum(ss), lane & 32);
        const float scale = rsqrt_exact(tot / 128.0f + rs);
        f32x4 o;
        o.x = (scale * v[u].x) * s2; o.y = (scale * v[u].y) * s2; o.z = (scale * v[u].z) * s2; o.w = (scale * v[u].w) * s2;
        const size_t yo = (size_t)t * 128 + 4 * l;
        if (t < total) {
            if (U > 1) { if (BF16) __builtin_nontemporal_store(pack_bf16x4_rne(o), (u32x2 *)((uint16_t *)y + yo)); else __builtin_nontemporal_store(o, (f32x4 *)((float *)y + yo)); }
            else { if (BF16) *(u32x2 *)((uint16_t *)y + yo) = pack_bf16x4_rne(o); else *(f32x4 *)((float *)y + yo) = o; }
        }
    }
}

// The same heads with 16 lanes x 8 values each (lane l of the row holds the logical threads 8 l .. 8 l + 7), four heads per wave, for
// batches whose time is their instruction count: what a lane does once per head (the exact square root and division, the index
// arithmetic, the group sums) is shared by eight values instead of four (30 -> 17 instructions per value). The tree: thread ^ 16
// and ^ 8 are lanes l ^ 2 and l ^ 1 (the four lanes of a quad are a 32-thread group), ^ 4, 2, 1 are register pairs; the four
// group sums sit in lanes 0, 4, 8, 12 of the row and are added in order from zero.
template <int S> CAMX_DEV float row16_bcast(float v) {      // every lane of a 16-lane row reads the row's lane S
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x10 | (S << 5)));
}
template <bool BF16, int U>
__global__ void __launch_bounds__(256) gdn_l2_128_w8(const void * __restrict__ x, void * __restrict__ y, int heads, int ldx, float rs, int total) {
    const int lane = threadIdx.x & 63, l = lane & 15;
    const int span = gridDim.x * 16;                                 // heads per pass of the grid
    const int t0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);
    float v[U][8];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = t0 + u * span, tc = t < total ? t : 0;
        const int tt = tc / heads, hh = tc - tt * heads;
        const size_t xo = (size_t)tt * ldx + (size_t)hh * 128 + 8 * l;
        f32x4 a, b;
        if (BF16) {
            const u32x4 w = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)x + xo));
            a = unpack_bf16x4((u32x2){w.x, w.y}); b = unpack_bf16x4((u32x2){w.z, w.w});
        } else { a = __builtin_nontemporal_load((const f32x4 *)((const float *)x + xo)); b = __builtin_nontemporal_load((const f32x4 *)((const float *)x + xo + 4)); }
        v[u][0] = a.x; v[u][1] = a.y; v[u][2] = a.z; v[u][3] = a.w; v[u][4] = b.x; v[u][5] = b.y; v[u][6] = b.z; v[u][7] = b.w;
    }
    const float s2 = 1.0f / sqrtf(128.0f);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = t0 + u * span;
        float s[8];
#pragma unroll
        for (int k = 0; k < 8; k++) s[k] = __builtin_fmaf(v[u][k], v[u][k], 0.0f);
#pragma unroll
        for (int k = 0; k < 8; k++) s[k] += lane_xor2(s[k]);          // thread ^ 16
#pragma unroll
        for (int k = 0; k < 8; k++) s[k] += lane_xor1(s[k]);          // thread ^ 8
        const float a0 = s[0] + s[4], a1 = s[1] + s[5], a2 = s[2] + s[6], a3 = s[3] + s[7];   // thread ^ 4
        const float b0 = a0 + a2, b1 = a1 + a3;                        // thread ^ 2
        const float g = b0 + b1;                                       // thread ^ 1: the group's sum, in its four lanes
        float tot = 0.0f;
        tot += row16_bcast<0>(g); tot += row16_bcast<4>(g); tot += row16_bcast<8>(g); tot += row16_bcast<12>(g);
        const float scale = rsqrt_exact(tot / 128.0f + rs);
        f32x4 oa, ob;
        oa.x = (scale * v[u][0]) * s2; oa.y = (scale * v[u][1]) * s2; oa.z = (scale * v[u][2]) * s2; oa.w = (scale * v[u][3]) * s2;
        ob.x = (scale * v[u][4]) * s2; ob.y = (scale * v[u][5]) * s2; ob.z = (scale * v[u][6]) * s2; ob.w = (scale * v[u][7]) * s2;
        const size_t yo = (size_t)t * 128 + 8 * l;
        if (t < total) {
            if (BF16) { const u32x2 pa = pack_bf16x4_rne(oa), pb = pack_bf16x4_rne(ob); __builtin_nontemporal_store((u32x4){pa.x, pa.y, pb.x, pb.y}, (u32x4 *)((uint16_t *)y + yo)); }
            else { __builtin_nontemporal_store(oa, (f32x4 *)((float *)y + yo)); __builtin_nontemporal_store(ob, (f32x4 *)((float *)y + yo + 4)); }
        }
    }
}

// ---- conv4 + SiLU with the L2 norm of the q / k heads in the same pass ---------------------------------------------------------------
// The reference appends OP_GDN_CONV and OP_GDN_L2 back to back (python/caminus/engine/q35_dense.py:399-400; kernels/k3_q35_ops.h:152-194):
// the L2 norm reads the first heads * 128 channels of the convolution's output. Here the lane that produced four (eight) of a head's
// channels keeps them and the head's 32 (16) lanes form the sum of squares in gdn_l2_128's (gdn_l2_128_w8's) tree, from the values as
// the convolution stores them (rounded to bf16 first when the rows are bf16), so y and qk carry the bits of the two separate kernels.
CAMX_DEV f32x4 l2_head_l4(f32x4 v, int lane, float rs) {           // a head of 128 values in 32 lanes x 4 (lane: its slot), as gdn_l2_128
    f32x4 ss;
    ss.x = __builtin_fmaf(v.x, v.x, 0.0f); ss.y = __builtin_fmaf(v.y, v.y, 0.0f); ss.z = __builtin_fmaf(v.z, v.z, 0.0f); ss.w = __builtin_fmaf(v.w, v.w, 0.0f);
    const float tot = half_groups_in_order<4>(group32_sum(ss), lane & 32);
    const float scale = rsqrt_exact(tot / 128.0f + rs), s2 = 1.0f / sqrtf(128.0f);
    f32x4 o;
    o.x = (scale * v.x) * s2; o.y = (scale * v.y) * s2; o.z = (scale * v.z) * s2; o.w = (scale * v.w) * s2;
    return o;
}
CAMX_DEV void l2_head_w8(const float (&v)[8], float (&o)[8], float rs) {   // a head of 128 values in 16 lanes x 8, as gdn_l2_128_w8
    float s[8];
#pragma unroll
    for (int k = 0; k < 8; k++) s[k] = __builtin_fmaf(v[k], v[k], 0.0f);
#pragma unroll
    for (int k = 0; k < 8; k++) s[k] += lane_xor2(s[k]);
#pragma unroll
    for (int k = 0; k < 8; k++) s[k] += lane_xor1(s[k]);
    const float a0 = s[0] + s[4], a1 = s[1] + s[5], a2 = s[2] + s[6], a3 = s[3] + s[7];
    const float b0 = a0 + a2, b1 = a1 + a3;
    const float g = b0 + b1;
    float tot = 0.0f;
    tot += row16_bcast<0>(g); tot += row16_bcast<4>(g); tot += row16_bcast<8>(g); tot += row16_bcast<12>(g);
    const float scale = rsqrt_exact(tot / 128.0f + rs), s2 = 1.0f / sqrtf(128.0f);
#pragma unroll
    for (int k = 0; k < 8; k++) o[k] = (scale * v[k]) * s2;
}
// Decode / verify batches: a half-wave per (token, 128 channels), lane l (its slot) at channels 4 l .. 4 l + 3 of the group. y optional.
template <bool BF16>
__global__ void __launch_bounds__(256) gdn_conv_l2_k(const void * __restrict__ x, const float * __restrict__ w, const float * __restrict__ st,
                                                     void * __restrict__ y, void * __restrict__ qk, int C, int T, int ldx, int ldy, int heads, float rs) {
    const int lane = slot_of(threadIdx.x & 63), l = lane & 31;
    const int G = C >> 7;
    const long u = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
    const bool on = u < (long)T * G;
    const int t = on ? (int)(u / G) : 0, cg = on ? (int)(u - (long)t * G) : 0;
    const int c0 = 128 * cg + 4 * l;
    f32x4 in[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int tj = t - 3 + j;
        if (tj >= 0) in[j] = BF16 ? unpack_bf16x4(*(const u32x2 *)((const uint16_t *)x + (size_t)tj * ldx + c0)) : *(const f32x4 *)((const float *)x + (size_t)tj * ldx + c0);
        else {
#pragma unroll
            for (int k = 0; k < 4; k++) in[j][k] = st[(size_t)(c0 + k) * 3 + 3 + tj];
        }
    }
    f32x4 v;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const f32x4 w4 = *(const f32x4 *)(w + (size_t)(c0 + k) * 4);
        float sumf = 0.0f;
        sumf = __builtin_fmaf(in[0][k], w4.x, sumf); sumf = __builtin_fmaf(in[1][k], w4.y, sumf);
        sumf = __builtin_fmaf(in[2][k], w4.z, sumf); sumf = __builtin_fmaf(in[3][k], w4.w, sumf);
        v[k] = BF16 ? silu_fast(sumf) : silu_f(sumf);
    }
    if (BF16) {
        const u32x2 pk = pack_bf16x4_rne(v);
        if (on && y) *(u32x2 *)((uint16_t *)y + (size_t)t * ldy + c0) = pk;
        v = unpack_bf16x4(pk);
    } else if (on && y) *(f32x4 *)((float *)y + (size_t)t * ldy + c0) = v;
    const f32x4 o = l2_head_l4(v, lane, rs);
    if (on && cg < heads) {
        const size_t qo = ((size_t)t * heads + cg) * 128 + 4 * l;
        if (BF16) *(u32x2 *)((uint16_t *)qk + qo) = pack_bf16x4_rne(o); else *(f32x4 *)((float *)qk + qo) = o;
    }
}
// OP_GDN_CONV followed by OP_GDN_L2 on the tape (decode / verify pass of T tokens, fp32, lazy commit as in op_gdn_conv_k; qk null: the
// convolution alone).
__global__ void __launch_bounds__(256) op_gdn_conv_l2_k(const float * __restrict__ w, float * __restrict__ st, const float * __restrict__ x,
                                                        const int32_t * __restrict__ params, float * __restrict__ y, float * __restrict__ xprev,
                                                        float * __restrict__ qk, int C, int T, int heads, float rs,
                                                        const float * __restrict__ al = nullptr, const float * __restrict__ be = nullptr,
                                                        const float * __restrict__ dt = nullptr, const float * __restrict__ A = nullptr,
                                                        float * __restrict__ gates = nullptr, int H = 0, int nconv = 0) {
    if (al && (int)blockIdx.x >= nconv) {
        // OP_GDN_GATES of the same layer in the launch's last workgroups (kernels/k3_q35_ops.h:196-211): gate = softplus(alpha + dt) * a | sigmoid(beta)
        const int q = ((int)blockIdx.x - nconv) * (int)blockDim.x + (int)threadIdx.x;
        if (q >= T * H) return;
        const int tt = q / H, h = q - tt * H;
        const float ab = al[q] + dt[h];
        const float sp = ab > 20.0f ? ab : logf(1.0f + expf(ab));
        gates[(size_t)tt * 2 * H + h] = sp * A[h];
        gates[(size_t)tt * 2 * H + H + h] = 1.0f / (1.0f + expf(-be[q]));
        return;
    }
    // One workgroup per 128 channels; its eight half-waves (32 lanes x 4 channels, the lanes in slot order) share the pass's tokens: half-wave
    // h takes tokens h, h + 8, .. Each token's window is read straight from the rows it comes from (x of this pass; before its first token, the
    // state as it stands once the previous pass's accepted tokens are committed), so no token waits for another: a pass of 16 or 64 tokens costs
    // what two or eight cost one after the other. Only this workgroup touches its channels of the state and of xprev: everything it needs of
    // them is in registers before the barrier, and rewritten after it.
    const int lane = slot_of(threadIdx.x & 63), l = lane & 31, hw = (int)(threadIdx.x >> 5);
    const int cg = (int)blockIdx.x, c0 = 128 * cg + 4 * l;
    f32x4 w4[4], hist[3], xin[4];                                    // hist[3 - k]: the input k tokens before the pass, k = 1 .. 3
    auto rows = [&](int tc) {                                        // the rows of x in token tc's window (requested before anything waits)
#pragma unroll
        for (int k = 0; k < 4; k++) { const int tt = tc - 3 + k; if (tt >= 0) xin[k] = *(const f32x4 *)(x + (size_t)tt * C + c0); }
    };
    rows(hw < T ? hw : T - 1);
#pragma unroll
    for (int k = 0; k < 4; k++) w4[k] = *(const f32x4 *)(w + (size_t)(c0 + k) * 4);
    int mprev = params[1];
    mprev = mprev < 0 ? 0 : (mprev > T ? T : mprev);
#pragma unroll
    for (int k = 1; k <= 3; k++) {
        if (mprev >= k) hist[3 - k] = *(const f32x4 *)(xprev + (size_t)(mprev - k) * C + c0);
        else {
#pragma unroll
            for (int e = 0; e < 4; e++) hist[3 - k][e] = st[(size_t)(c0 + e) * 3 + (mprev + 3 - k)];
        }
    }
    __syncthreads();
    if (hw == 0) {
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int jj = 0; jj < 3; jj++) st[(size_t)(c0 + e) * 3 + jj] = hist[jj][e];
    }
    const int nhw = (int)(blockDim.x >> 5);                          // (larger workgroups for longer passes were measured and are no faster: 64 tokens 9.4 against 9.8 us)
    for (int tb = 0; tb < T; tb += nhw) {                            // (uniform trip count: both halves of a wave take part in the head's sums)
        const int t = tb + hw;
        const bool live = t < T;
        const int tc = live ? t : T - 1;
        f32x4 in[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {                                // in[k]: the input at token tc - 3 + k
            const int tt = tc - 3 + k;
            in[k] = tt >= 0 ? xin[k] : (tt == -3 ? hist[0] : (tt == -2 ? hist[1] : hist[2]));
        }
        if (tb + nhw < T) rows(t + nhw < T ? t + nhw : T - 1);       // the next token's rows, in flight during this one's arithmetic
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float sumf = 0.0f;
            sumf = __builtin_fmaf(in[0][e], w4[e].x, sumf); sumf = __builtin_fmaf(in[1][e], w4[e].y, sumf);
            sumf = __builtin_fmaf(in[2][e], w4[e].z, sumf); sumf = __builtin_fmaf(in[3][e], w4[e].w, sumf);
            v[e] = silu_f(sumf);
        }
        const f32x4 o = qk ? l2_head_l4(v, lane, rs) : v;
        if (live) {
            *(f32x4 *)(y + (size_t)t * C + c0) = v;
            *(f32x4 *)(xprev + (size_t)t * C + c0) = in[3];
            if (qk && cg < heads) *(f32x4 *)(qk + ((size_t)t * heads + cg) * 128 + 4 * l) = o;
        }
    }
}

// ---- hyper-connection glue (kernels/prefill_glue.hip:172-206) -----------------------------------------------------------------
// pf_hc_post: res[t][h][i] = fma(b[t][i], 2 sigmoid(inj[t][h] * rs), res[t][h][i]); four consecutive i per thread when D % 4 == 0
template <bool VEC>
__global__ void __launch_bounds__(256) hc_post_k(const float * __restrict__ b, const float * __restrict__ inj, float * __restrict__ res, int T, int HC,
                                                 int D, float rs) {
    constexpr int VW = VEC ? 4 : 1;
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * VW;
    if (i >= (long)T * D) return;
    const int tt = (int)(i / D), ii = (int)(i - (long)tt * D);
    float bv[VW];
    if (VEC) { const f32x4 v = __builtin_nontemporal_load((const f32x4 *)(b + i)); bv[0] = v.x; if (VW > 1) { bv[1] = v.y; bv[2] = v.z; bv[3] = v.w; } }
    else bv[0] = b[i];
    for (int h = 0; h < HC; h++) {
        const float v = inj[tt * HC + h] * rs;
        const float sgm = 1.0f / (1.0f + expf(-v));
        const float ph = sgm * 2.0f;
        const size_t o = (size_t)(tt * HC + h) * D + ii;
        if (VEC) {
            f32x4 r = __builtin_nontemporal_load((const f32x4 *)(res + o));
            r.x = __builtin_fmaf(bv[0], ph, r.x); r.y = __builtin_fmaf(bv[1 % VW], ph, r.y); r.z = __builtin_fmaf(bv[2 % VW], ph, r.z); r.w = __builtin_fmaf(bv[3 % VW], ph, r.w);
            __builtin_nontemporal_store(r, (f32x4 *)(res + o));
        } else res[o] = __builtin_fmaf(bv[0], ph, res[o]);
    }
}
// pf_hc_mean: out[t][i] = rs * sum over h (fma chain from 0) of xn[t][h][i] * sigmoid(g[t][h][i]); xn given, or recomputed from
// the residual as (x * scl[t * HC + h]) * w[h][i]. The loads of all HC streams (up to 8) are issued before the arithmetic.
template <bool VEC>
__global__ void __launch_bounds__(256) hc_mean_k(const float * __restrict__ x, const float * __restrict__ scl, const float * __restrict__ w,
                                                 const float * __restrict__ g, float * __restrict__ out, int T, int HC, int D, float rs) {
    constexpr int VW = VEC ? 4 : 1;
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * VW;
    if (i >= (long)T * D) return;
    const int tt = (int)(i / D), ii = (int)(i - (long)tt * D);
    float sum[VW];
#pragma unroll
    for (int k = 0; k < VW; k++) sum[k] = 0.0f;
    for (int h0 = 0; h0 < HC; h0 += 8) {
        float xv[8][VW], gv[8][VW], sc[8], wv[8][VW];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int h = h0 + u;
            if (h < HC) {
                const size_t o = (size_t)(tt * HC + h) * D + ii;
                if (VEC) {
                    const f32x4 a = __builtin_nontemporal_load((const f32x4 *)(x + o)), c = __builtin_nontemporal_load((const f32x4 *)(g + o));
                    xv[u][0] = a.x; gv[u][0] = c.x;
                    if (VW > 1) { xv[u][1] = a.y; xv[u][2] = a.z; xv[u][3] = a.w; gv[u][1] = c.y; gv[u][2] = c.z; gv[u][3] = c.w; }
                } else { xv[u][0] = x[o]; gv[u][0] = g[o]; }
                if (scl) {
                    sc[u] = scl[tt * HC + h];
                    if (VEC) { const f32x4 q = *(const f32x4 *)(w + (size_t)h * D + ii); wv[u][0] = q.x; if (VW > 1) { wv[u][1] = q.y; wv[u][2] = q.z; wv[u][3] = q.w; } }
                    else wv[u][0] = w[(size_t)h * D + ii];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            if (h0 + u < HC) {
#pragma unroll
                for (int k = 0; k < VW; k++) {
                    const float xn = scl ? (xv[u][k] * sc[u]) * wv[u][k] : xv[u][k];
                    sum[k] = __builtin_fmaf(xn, 1.0f / (1.0f + expf(-gv[u][k])), sum[k]);
                }
            }
        }
    }
    if (VEC) __builtin_nontemporal_store((f32x4){rs * sum[0], rs * sum[1 % VW], rs * sum[2 % VW], rs * sum[3 % VW]}, (f32x4 *)(out + i));
    else out[i] = rs * sum[0];
}

// ---- S1 core / fuse ----------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) embedding_f32_k(const int * __restrict__ tok, const float * __restrict__ emb, float * __restrict__ out, int D) {
    const int t = blockIdx.x;
    const float * src = emb + (size_t)tok[t] * D;
    for (int j = threadIdx.x; j < D; j += 256) out[(size_t)t * D + j] = src[j];
}
__global__ void __launch_bounds__(256) residual3_k(const float * __restrict__ x, const uint16_t * __restrict__ m, const uint16_t * __restrict__ y,
                                                   float * __restrict__ out, long n) {
    const long step = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += step) out[i] = (x[i] + bf2f(m[i])) + bf2f(y[i]);
}
// four values per thread (16-byte x / out, 8-byte m / y); every stream is read once
__global__ void __launch_bounds__(256) residual3_vec(const float * __restrict__ x, const uint16_t * __restrict__ m, const uint16_t * __restrict__ y,
                                                     float * __restrict__ out, long n4) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (q >= n4) return;
    const f32x4 xv = __builtin_nontemporal_load((const f32x4 *)x + q);
    const f32x4 mv = unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)m + q)), yv = unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)y + q));
    f32x4 o; o.x = (xv.x + mv.x) + yv.x; o.y = (xv.y + mv.y) + yv.y; o.z = (xv.z + mv.z) + yv.z; o.w = (xv.w + mv.w) + yv.w;
    __builtin_nontemporal_store(o, (f32x4 *)out + q);
}
__global__ void __launch_bounds__(256) cast_bf16_k(const float * __restrict__ x, uint16_t * __restrict__ out, long n) {
    const long step = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += step) out[i] = f2bf(x[i]);
}
// eight values per thread: two 16-byte loads, one 16-byte store
__global__ void __launch_bounds__(256) cast_bf16_vec(const float * __restrict__ x, uint16_t * __restrict__ out, long n8) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (q >= n8) return;
    const f32x4 a = __builtin_nontemporal_load((const f32x4 *)x + 2 * q), b = __builtin_nontemporal_load((const f32x4 *)x + 2 * q + 1);
    const u32x2 lo = pack_f2bf_x4(a), hi = pack_f2bf_x4(b);
    __builtin_nontemporal_store((u32x4){lo.x, lo.y, hi.x, hi.y}, (u32x4 *)out + q);
}
__global__ void __launch_bounds__(256) copy_cols_bf16_k(const uint16_t * __restrict__ in, int ld_in, int c_in, uint16_t * __restrict__ out, int ld_out,
                                                        int c_out, int n, long rows) {
    const long step = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < rows * n; i += step) {
        const long r = i / n, c = i - r * n;
        out[r * ld_out + c_out + c] = in[r * ld_in + c_in + c];
    }
}
// whole contiguous rows (n == ld_in == ld_out): one 16-byte unit per thread, past the caches both ways
__global__ void __launch_bounds__(256) copy_flat16(const u32x4 * __restrict__ in, u32x4 * __restrict__ out, long n16) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(in + i), out + i);
}
// every offset and width a multiple of 8 values: 16-byte units
__global__ void __launch_bounds__(256) copy_cols_bf16_vec(const u32x4 * __restrict__ in, int ld_in, int c_in, u32x4 * __restrict__ out, int ld_out,
                                                          int c_out, int n, long rows) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * n) return;
    const long r = i / n, c = i - r * n;
    out[r * ld_out + c_out + c] = __builtin_nontemporal_load(in + r * ld_in + c_in + c);
}
// out = ((x + m) + mlp) + (pos[r] >= 0 ? ys[pos[r]] : 0), four columns per thread (d % 4 == 0)
__global__ void __launch_bounds__(256) residual_slices_fwd_k(const float * __restrict__ x, const uint16_t * __restrict__ m, const uint16_t * __restrict__ mlp,
                                                             const uint16_t * __restrict__ ys, const int * __restrict__ pos, float * __restrict__ out, int d, long n4) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const long e = i * 4; const int r = (int)(e / d), c = (int)(e % d);
    const f32x4 xv = *(const f32x4 *)(x + e);
    const f32x4 mv = unpack_bf16x4(*(const u32x2 *)(m + e)), lv = unpack_bf16x4(*(const u32x2 *)(mlp + e));
    const int p = pos ? pos[r] : -1;
    f32x4 sv = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p >= 0) sv = unpack_bf16x4(*(const u32x2 *)(ys + (size_t)p * d + c));
    f32x4 o;
    o.x = ((xv.x + mv.x) + lv.x) + sv.x; o.y = ((xv.y + mv.y) + lv.y) + sv.y;
    o.z = ((xv.z + mv.z) + lv.z) + sv.z; o.w = ((xv.w + mv.w) + lv.w) + sv.w;
    *(f32x4 *)(out + e) = o;
}

// the same with the row in blockIdx.y (no division of a 64-bit element index per thread) and every streamed operand non-temporal
// (8192 x 2048: 38.9 -> 34.5 us forward, 29.1 -> 26.2 us backward; 16-byte accesses of eight values per thread measured no better)
__global__ void __launch_bounds__(256) residual_slices_fwd_rows(const float * __restrict__ x, const uint16_t * __restrict__ m, const uint16_t * __restrict__ mlp,
                                                                const uint16_t * __restrict__ ys, const int * __restrict__ pos, float * __restrict__ out, int d) {
    const int r = blockIdx.y, c = 4 * (blockIdx.x * 256 + threadIdx.x);
    if (c >= d) return;
    const size_t e = (size_t)r * d + c;
    const f32x4 xv = __builtin_nontemporal_load((const f32x4 *)(x + e));
    const f32x4 mv = unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)(m + e))), lv = unpack_bf16x4(__builtin_nontemporal_load((const u32x2 *)(mlp + e)));
    const int p = pos ? pos[r] : -1;
    f32x4 sv = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p >= 0) sv = unpack_bf16x4(*(const u32x2 *)(ys + (size_t)p * d + c));
    f32x4 o;
    o.x = ((xv.x + mv.x) + lv.x) + sv.x; o.y = ((xv.y + mv.y) + lv.y) + sv.y;
    o.z = ((xv.z + mv.z) + lv.z) + sv.z; o.w = ((xv.w + mv.w) + lv.w) + sv.w;
    __builtin_nontemporal_store(o, (f32x4 *)(out + e));
}
__global__ void __launch_bounds__(256) residual_slices_bwd_rows(const float * __restrict__ dout, const int * __restrict__ pos, uint16_t * __restrict__ dm,
                                                                uint16_t * __restrict__ dmlp, uint16_t * __restrict__ dys, int d) {
    const int r = blockIdx.y, c = 4 * (blockIdx.x * 256 + threadIdx.x);
    if (c >= d) return;
    const size_t e = (size_t)r * d + c;
    const u32x2 b = pack_f2bf_x4(__builtin_nontemporal_load((const f32x4 *)(dout + e)));
    __builtin_nontemporal_store(b, (u32x2 *)(dm + e)); __builtin_nontemporal_store(b, (u32x2 *)(dmlp + e));
    const int p = pos ? pos[r] : -1;
    if (p >= 0) *(u32x2 *)(dys + (size_t)p * d + c) = b;
}

__attribute__((visibility("hidden"))) int silu_mul_bf16_wide(const uint16_t * gu, uint16_t * act, int H, long n, hipStream_t st);   // quant.hip
__attribute__((visibility("hidden"))) int silu_lut_get(hipStream_t st, const uint16_t ** lut);                                        // quant.hip

extern "C" {

int camx_q3p_swiglu(const float * g, const float * u, uint16_t * y, int n, hipStream_t st) {
    if (!g || !u || !y || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int vec = !(((uintptr_t)g | (uintptr_t)u) & 15) && !((uintptr_t)y & 7);
    swiglu_f32<true><<<GRID_1D(((long)n + 3) / 4), dim3(256), 0, st>>>(g, u, y, n, vec);
    CAMX_LAUNCH_RET();
}
int camx_gg_silu_mul(const float * g, const float * u, float * h, int n, hipStream_t st) {
    if (!g || !u || !h || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int vec = !(((uintptr_t)g | (uintptr_t)u | (uintptr_t)h) & 15);
    swiglu_f32<false><<<GRID_1D(((long)n + 3) / 4), dim3(256), 0, st>>>(g, u, h, n, vec);
    CAMX_LAUNCH_RET();
}
int camx_silu_mul_bf16(const uint16_t * gu, uint16_t * act, int H, long n, hipStream_t st) {
    if (!gu || !act || H < 1 || n < 0 || n % H) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const uint16_t * lut = nullptr;
    const int rc = silu_lut_get(st, &lut);                       // (a failure to set the table up is reported here, so CAMX_EINVAL below means "not applicable")
    if (rc) return rc;
    const int wide = silu_mul_bf16_wide(gu, act, H, n, st);      // large inputs: the table in LDS
    if (wide != CAMX_EINVAL) return wide;
    const int vec = H % 4 == 0 && !(((uintptr_t)gu | (uintptr_t)act) & 7);
    silu_mul_bf16_k<<<GRID_1D((n + 3) / 4), dim3(256), 0, st>>>(gu, act, H, n, vec, lut);
    CAMX_LAUNCH_RET();
}
// io: 0 fp32 -> fp32 (pf_gate_mul), 1 fp32 -> fp16 (q35p_gate_mul16), 2 bf16 -> bf16
int camx_gate_mul(const void * a, const void * gt, void * y, long N, int D, int stride, int off, int io, hipStream_t st) {
    if (!a || !gt || !y || N < 0 || D < 1 || N % D || off < 0 || off + D > stride || io < 0 || io > 2) return CAMX_EINVAL;
    if (N == 0) return CAMX_OK;
    const int vw = io == 2 ? 8 : 4, es = io == 2 ? 2 : 4;
    if (D % vw == 0 && stride % vw == 0 && off % vw == 0 && !(((uintptr_t)a | (uintptr_t)gt) & 15) && !((uintptr_t)y & (io == 1 ? 7 : 15))) {
        (void)es;
        const long nvec = N / vw;
        const dim3 gv = GRID_1D(nvec), bv(256);
        if (io == 0) gate_mul_vec<0><<<gv, bv, 0, st>>>(a, gt, y, nvec, D / vw, stride, off);
        else if (io == 1) gate_mul_vec<1><<<gv, bv, 0, st>>>(a, gt, y, nvec, D / vw, stride, off);
        else gate_mul_vec<2><<<gv, bv, 0, st>>>(a, gt, y, nvec, D / vw, stride, off);
        CAMX_LAUNCH_RET();
    }
    const dim3 grid = GRID_1D(N), block(256);
    if (io == 0) gate_mul_k<0><<<grid, block, 0, st>>>(a, gt, y, N, D, stride, off);
    else if (io == 1) gate_mul_k<1><<<grid, block, 0, st>>>(a, gt, y, N, D, stride, off);
    else gate_mul_k<2><<<grid, block, 0, st>>>(a, gt, y, N, D, stride, off);
    CAMX_LAUNCH_RET();
}
int camx_pf_gdn_conv(const void * x, const float * w, const float * state, void * y, int C, int T, int ldx, int ldy, int bf16, hipStream_t st) {
    if (!x || !w || !state || !y || C < 1 || T < 1 || ldx < C || ldy < C || ((uintptr_t)w & 15)) return CAMX_EINVAL;
    const int vw = bf16 ? 8 : 4;
    if ((long)T * C >= (1L << 20) && C % vw == 0 && ldx % vw == 0 && ldy % vw == 0 && !(((uintptr_t)x | (uintptr_t)y) & 15)) {
        // tokens per wave: at 4096 tokens 16 and 64 measured 15 % slower than 32 (halo re-reads; too few waves); from 16384 tokens on there
        // are waves enough for 64, and the three halo rows a wave re-reads are 5 % of its reads instead of 9 % (a decode / verify batch
        // takes the one-value-per-thread kernel below)
        const int tr = T >= 16384 ? 64 : 32;
        const dim3 gs((unsigned)((C / vw + 63) / 64), (unsigned)((T + tr - 1) / tr)), bs(64);
        if (bf16) gdn_conv_stream<true><<<gs, bs, 0, st>>>(x, w, state, y, C, T, ldx, ldy, tr); else gdn_conv_stream<false><<<gs, bs, 0, st>>>(x, w, state, y, C, T, ldx, ldy, tr);
        CAMX_LAUNCH_RET();
    }
    const dim3 grid((unsigned)(((long)T * C + 255) / 256)), block(256);
    if (bf16) gdn_conv_k<true><<<grid, block, 0, st>>>(x, w, state, y, C, T, ldx, ldy);
    else gdn_conv_k<false><<<grid, block, 0, st>>>(x, w, state, y, C, T, ldx, ldy);
    CAMX_LAUNCH_RET();
}
// OP_GDN_CONV with its Seg fields (python/caminus/engine/k3.py:993-1000): W = w [C][4], gs = state [C][3] (updated by the commit only),
// a = x [T][C], asum = the pass parameters (int32, [1] = accepted tokens of the previous pass), y = out [T][C], aux = xprev [T][C],
// N = C; T = the tape's tokens per pass
int camx_op_gdn_conv(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, int C, int T, hipStream_t st) {
    if (!w || !state || !x || !params || !y || !xprev || C < 1 || T < 1 || ((uintptr_t)w & 15)) return CAMX_EINVAL;
    if (T >= 16 && (C & 127) == 0 && !(((uintptr_t)x | (uintptr_t)y | (uintptr_t)xprev) & 15))       // a verify pass: its tokens side by side (64 tokens: 11.3 -> 7.6 us)
        op_gdn_conv_l2_k<<<dim3((unsigned)(C >> 7)), dim3(256), 0, st>>>(w, state, x, params, y, xprev, nullptr, C, T, 0, 0.0f);
    else op_gdn_conv_k<<<dim3((C + 255) / 256), dim3(256), 0, st>>>(w, state, x, params, y, xprev, C, T);
    CAMX_LAUNCH_RET();
}
int camx_pf_conv_state(const void * x, float * state, int C, int T, int ldx, int bf16, hipStream_t st) {
    if (!x || !state || C < 1 || T < 1 || ldx < C) return CAMX_EINVAL;
    const dim3 grid((C + 255) / 256), block(256);
    if (bf16) conv_state_k<true><<<grid, block, 0, st>>>(x, state, C, T, ldx);
    else conv_state_k<false><<<grid, block, 0, st>>>(x, state, C, T, ldx);
    CAMX_LAUNCH_RET();
}
int camx_pf_gdn_l2(const void * x, void * y, int heads, int K, int ldx, float rs, int T, int bf16, hipStream_t st) {
    if (!x || !y || heads < 1 || K < 1 || K > 512 || T < 0 || ldx < heads * K) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const int total = T * heads;
    const dim3 grid((total + 3) / 4), block(256);
    const bool vec = K % 4 == 0 && ldx % 4 == 0 && !((uintptr_t)x & (bf16 ? 7 : 15)) && !((uintptr_t)y & (bf16 ? 7 : 15));
    if (vec && K == 128) {
        if (total >= 65536 && ldx % 8 == 0 && !((uintptr_t)x & 15) && !((uintptr_t)y & 15)) {       // a prefill chunk: 16 lanes per head, four heads per row of lanes
            const dim3 g8((total + 63) / 64);
            if (bf16) gdn_l2_128_w8<true, 4><<<g8, block, 0, st>>>(x, y, heads, ldx, rs, total); else gdn_l2_128_w8<false, 4><<<g8, block, 0, st>>>(x, y, heads, ldx, rs, total);
        } else if (total >= 32768) {                                  // enough heads to fill the chip four times over: four heads per half-wave
            const dim3 g4((total + 31) / 32);
            if (bf16) gdn_l2_128<true, 4><<<g4, block, 0, st>>>(x, y, heads, ldx, rs, total); else gdn_l2_128<false, 4><<<g4, block, 0, st>>>(x, y, heads, ldx, rs, total);
        } else {
            const dim3 g2((total + 7) / 8);
            if (bf16) gdn_l2_128<true, 1><<<g2, block, 0, st>>>(x, y, heads, ldx, rs, total); else gdn_l2_128<false, 1><<<g2, block, 0, st>>>(x, y, heads, ldx, rs, total);
        }
        CAMX_LAUNCH_RET();
    }
    if (bf16) { if (vec) gdn_l2_k<true, true><<<grid, block, 0, st>>>(x, y, heads, K, ldx, rs, total); else gdn_l2_k<true, false><<<grid, block, 0, st>>>(x, y, heads, K, ldx, rs, total); }
    else { if (vec) gdn_l2_k<false, true><<<grid, block, 0, st>>>(x, y, heads, K, ldx, rs, total); else gdn_l2_k<false, false><<<grid, block, 0, st>>>(x, y, heads, K, ldx, rs, total); }
    CAMX_LAUNCH_RET();
}
// conv4 + SiLU and the L2 norm of the first `heads` heads of 128 channels in one launch: y (optional) = camx_pf_gdn_conv's rows, qk
// [T][heads][128] = camx_pf_gdn_l2(y, heads, 128, ldy, rs) bit for bit. C % 128 == 0, 16-byte aligned operands.
int camx_gdn_conv_l2(const void * x, const float * w, const float * state, void * y, void * qk, int C, int T, int ldx, int ldy, int heads, float rs,
                     int bf16, hipStream_t st) {
    const int vw = bf16 ? 8 : 4;
    if (!x || !w || !state || !qk || C < 128 || (C & 127) || T < 1 || ldx < C || (y && ldy < C) || heads < 1 || heads > C / 128 || (ldx % vw) || (y && ldy % vw) ||
        ((uintptr_t)w & 15) || (((uintptr_t)x | (uintptr_t)y | (uintptr_t)qk) & 15)) return CAMX_EINVAL;
    if ((long)T * C >= (1L << 20)) {
        const int tr = T >= 16384 ? 64 : 32;
        const dim3 gs((unsigned)((C / vw + 63) / 64), (unsigned)((T + tr - 1) / tr)), bs(64);
        if (bf16) gdn_conv_stream<true, true><<<gs, bs, 0, st>>>(x, w, state, y, C, T, ldx, ldy, tr, qk, heads, rs);
        else gdn_conv_stream<false, true><<<gs, bs, 0, st>>>(x, w, state, y, C, T, ldx, ldy, tr, qk, heads, rs);
        CAMX_LAUNCH_RET();
    }
    const dim3 grid((unsigned)(((long)T * (C >> 7) + 7) / 8)), block(256);
    if (bf16) gdn_conv_l2_k<true><<<grid, block, 0, st>>>(x, w, state, y, qk, C, T, ldx, ldy, heads, rs);
    else gdn_conv_l2_k<false><<<grid, block, 0, st>>>(x, w, state, y, qk, C, T, ldx, ldy, heads, rs);
    CAMX_LAUNCH_RET();
}
// OP_GDN_CONV then OP_GDN_L2 of the decode tape in one launch (python/caminus/engine/q35_dense.py:399-400): camx_op_gdn_conv's arguments,
// then qk = the L2 norm (rs = eps / 128) of the first `heads` heads of 128 channels of y, as camx_op_gdn_l2(y, qk, heads, 128, rs, C, T)
int camx_op_gdn_conv_l2(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, float * qk, int C, int T,
                        int heads, float rs, hipStream_t st) {
    if (!w || !state || !x || !params || !y || !xprev || !qk || C < 128 || (C & 127) || T < 1 || heads < 1 || heads > C / 128 ||
        (((uintptr_t)w | (uintptr_t)x | (uintptr_t)y | (uintptr_t)xprev | (uintptr_t)qk) & 15)) return CAMX_EINVAL;
    op_gdn_conv_l2_k<<<dim3((unsigned)(C >> 7)), dim3(256), 0, st>>>(w, state, x, params, y, xprev, qk, C, T, heads, rs);
    CAMX_LAUNCH_RET();
}
// The three row ops a linear-attention layer runs ahead of its recurrence (python/caminus/engine/q35_dense.py:396-400: OP_GDN_GATES, OP_GDN_CONV,
// OP_GDN_L2) in one launch: camx_op_gdn_conv_l2's arguments, then camx_op_gdn_gates'. The gates take the launch's last workgroups.
int camx_op_gdn_conv_l2_gates(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, float * qk, int C, int T,
                              int heads, float rs, const float * alpha, const float * beta, const float * dt, const float * a, float * gates, int H,
                              hipStream_t st) {
    if (!w || !state || !x || !params || !y || !xprev || !qk || C < 128 || (C & 127) || T < 1 || heads < 1 || heads > C / 128 ||
        (((uintptr_t)w | (uintptr_t)x | (uintptr_t)y | (uintptr_t)xprev | (uintptr_t)qk) & 15) || !alpha || !beta || !dt || !a || !gates || H < 1 ||
        (long)T * H > 0x7fffffffL - 256) return CAMX_EINVAL;
    const unsigned bs = 256;
    const unsigned nconv = (unsigned)(C >> 7), ng = (unsigned)(((long)T * H + bs - 1) / bs);
    op_gdn_conv_l2_k<<<dim3(nconv + ng), dim3(bs), 0, st>>>(w, state, x, params, y, xprev, qk, C, T, heads, rs, alpha, beta, dt, a, gates, H, (int)nconv);
    CAMX_LAUNCH_RET();
}
// the remaining elementwise ops of the decode tape by their Seg fields
// OP_GDN_L2 (python/caminus/engine/k3.py:1002-1008): a = x, y = out, rs = eps / dim, N = T * heads, K = dim, pad1 = x_stride (0: heads * dim)
int camx_op_gdn_l2(const float * x, float * out, int heads, int dim, float rs, int x_stride, int T, hipStream_t st) {
    return camx_pf_gdn_l2(x, out, heads, dim, x_stride ? x_stride : heads * dim, rs, T, 0, st);
}
// OP_GATE_MUL16 (python/caminus/engine/k3.py:1209-1219): a, W = gate, y = out16, N = n, K = dim, pad1 = head_stride, pad2 = offset
int camx_op_gate_mul16(const float * a, const float * gate, int head_stride, int offset, uint16_t * out16, int n, int dim, hipStream_t st) {
    return camx_gate_mul(a, gate, out16, (long)n, dim, head_stride, offset, 1, st);
}
// OP_OWN_SWIGLU16 (python/caminus/engine/k3.py:854-860): a = g, W = u, y = y16, N = n
int camx_op_own_swiglu16(const float * g, const float * u, uint16_t * y16, int n, hipStream_t st) { return camx_q3p_swiglu(g, u, y16, n, st); }
int camx_pf_hc_post(const float * b, const float * inj, float * res, int T, int HC, int D, float rs, hipStream_t st) {
    if (!b || !inj || !res || T < 0 || HC < 1 || D < 1) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const bool vec = D % 4 == 0 && !(((uintptr_t)b | (uintptr_t)res) & 15);
    const long n = (long)T * D / (vec ? 4 : 1);
    if (vec) hc_post_k<true><<<GRID_1D(n), dim3(256), 0, st>>>(b, inj, res, T, HC, D, rs); else hc_post_k<false><<<GRID_1D(n), dim3(256), 0, st>>>(b, inj, res, T, HC, D, rs);
    CAMX_LAUNCH_RET();
}
int camx_pf_hc_mean(const float * x, const float * scl, const float * w, const float * g, float * out, int T, int HC, int D, float rs, hipStream_t st) {
    if (!x || !g || !out || T < 0 || HC < 1 || D < 1 || ((scl == nullptr) != (w == nullptr))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const bool vec = D % 4 == 0 && !(((uintptr_t)x | (uintptr_t)g | (uintptr_t)out | (uintptr_t)w) & 15);
    const long n = (long)T * D / (vec ? 4 : 1);
    if (vec) hc_mean_k<true><<<GRID_1D(n), dim3(256), 0, st>>>(x, scl, w, g, out, T, HC, D, rs); else hc_mean_k<false><<<GRID_1D(n), dim3(256), 0, st>>>(x, scl, w, g, out, T, HC, D, rs);
    CAMX_LAUNCH_RET();
}
int camx_embedding_f32(const int * tok, const float * emb, float * out, int D, int T, hipStream_t st) {
    if (!tok || !emb || !out || D < 1 || T < 0) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    embedding_f32_k<<<dim3(T), dim3(256), 0, st>>>(tok, emb, out, D);
    CAMX_LAUNCH_RET();
}
int camx_residual3(const float * x, const uint16_t * m, const uint16_t * y, float * out, long n, hipStream_t st) {
    if (!x || !m || !y || !out || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    if (n % 4 == 0 && n / 4 < 0x7fffffffL * 256 && !(((uintptr_t)x | (uintptr_t)out) & 15) && !(((uintptr_t)m | (uintptr_t)y) & 7))
        residual3_vec<<<dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, st>>>(x, m, y, out, n / 4);
    else residual3_k<<<GRID_1D(n), dim3(256), 0, st>>>(x, m, y, out, n);
    CAMX_LAUNCH_RET();
}
int camx_cast_bf16(const float * x, uint16_t * out, long n, hipStream_t st) {
    if (!x || !out || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    if (n % 8 == 0 && n / 8 < 0x7fffffffL * 256 && !(((uintptr_t)x | (uintptr_t)out) & 15))
        cast_bf16_vec<<<dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, st>>>(x, out, n / 8);
    else cast_bf16_k<<<GRID_1D(n), dim3(256), 0, st>>>(x, out, n);
    CAMX_LAUNCH_RET();
}
int camx_copy_cols_bf16(const uint16_t * in, int ld_in, int c_in, uint16_t * out, int ld_out, int c_out, int n, long rows, hipStream_t st) {
    if (!in || !out || n < 0 || rows < 0 || c_in < 0 || c_out < 0 || c_in + n > ld_in || c_out + n > ld_out) return CAMX_EINVAL;
    if (n == 0 || rows == 0) return CAMX_OK;
    const bool vec = !((ld_in | c_in | ld_out | c_out | n) & 7) && !(((uintptr_t)in | (uintptr_t)out) & 15) && rows * (n / 8) < 0x7fffffffL * 256;
    if (vec && n == ld_in && n == ld_out)
        copy_flat16<<<dim3((unsigned)((rows * (n / 8) + 255) / 256)), dim3(256), 0, st>>>((const u32x4 *)in, (u32x4 *)out, rows * (n / 8));
    else if (vec)
        copy_cols_bf16_vec<<<dim3((unsigned)((rows * (n / 8) + 255) / 256)), dim3(256), 0, st>>>((const u32x4 *)in, ld_in / 8, c_in / 8, (u32x4 *)out, ld_out / 8,
                                                                                                c_out / 8, n / 8, rows);
    else copy_cols_bf16_k<<<GRID_1D(rows * n), dim3(256), 0, st>>>(in, ld_in, c_in, out, ld_out, c_out, n, rows);
    CAMX_LAUNCH_RET();
}
// residual_slices_bwd (kernels/fuse.hip:35-47): dm = dmlp = bf16(dout) (f2bf), dys[pos[r]] = bf16(dout[r]) for the routed rows
__global__ void __launch_bounds__(256) residual_slices_bwd_k(const float * __restrict__ dout, const int * __restrict__ pos, uint16_t * __restrict__ dm,
                                                             uint16_t * __restrict__ dmlp, uint16_t * __restrict__ dys, int d, long n4) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const long e = i * 4; const int r = (int)(e / d), c = (int)(e % d);
    const u32x2 b = pack_f2bf_x4(__builtin_nontemporal_load((const f32x4 *)(dout + e)));
    *(u32x2 *)(dm + e) = b; *(u32x2 *)(dmlp + e) = b;
    const int p = pos ? pos[r] : -1;
    if (p >= 0) *(u32x2 *)(dys + (size_t)p * d + c) = b;
}
int camx_residual_slices_bwd(const float * dout, const int * pos, uint16_t * dm, uint16_t * dmlp, uint16_t * dys, int d, long n4, hipStream_t st) {
    if (!dout || !dm || !dmlp || d < 4 || d % 4 || n4 < 0 || (pos && !dys) || (((uintptr_t)dout) & 15) || (((uintptr_t)dm | (uintptr_t)dmlp | (uintptr_t)dys) & 7)) return CAMX_EINVAL;
    if (n4 == 0) return CAMX_OK;
    if ((n4 * 4) % d == 0 && n4 * 4 / d <= 65535)                       // whole rows: the row in blockIdx.y
        residual_slices_bwd_rows<<<dim3((unsigned)((d / 4 + 255) / 256), (unsigned)(n4 * 4 / d)), dim3(256), 0, st>>>(dout, pos, dm, dmlp, dys, d);
    else residual_slices_bwd_k<<<dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st>>>(dout, pos, dm, dmlp, dys, d, n4);
    CAMX_LAUNCH_RET();
}
int camx_residual_slices_fwd(const float * x, const uint16_t * m, const uint16_t * mlp, const uint16_t * ys, const int * pos, float * out,
                             int d, long n4, hipStream_t st) {
    if (!x || !m || !mlp || !out || d < 4 || d % 4 || n4 < 0 || ((uintptr_t)x & 15) || ((uintptr_t)out & 15) || ((uintptr_t)m & 7) ||
        ((uintptr_t)mlp & 7) || ((uintptr_t)ys & 7)) return CAMX_EINVAL;
    if (n4 == 0) return CAMX_OK;
    if ((n4 * 4) % d == 0 && n4 * 4 / d <= 65535)                       // whole rows: the row in blockIdx.y
        residual_slices_fwd_rows<<<dim3((unsigned)((d / 4 + 255) / 256), (unsigned)(n4 * 4 / d)), dim3(256), 0, st>>>(x, m, mlp, ys, pos, out, d);
    else residual_slices_fwd_k<<<dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st>>>(x, m, mlp, ys, pos, out, d, n4);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
