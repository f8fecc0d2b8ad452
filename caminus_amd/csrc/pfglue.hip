// More row kernels of the batched prefill for gfx950: the gated RMSNorm of the GDN output, the GDN gates, the fp16 KV
// append, the residual sums and bf16 operand copies of the glue, the hyper-connection average, and the per-layer-embedding
// gate / dilated conv / history. Replaces pf_gdn_norm and pf_gdn_gates (kernels/prefill_gdn.hip:80-92, 385-407),
// q35p_gdn_norm16 and q35p_kv_append16 (kernels/q35_prefill.hip:671-707), pf_ple_gate, pf_ple_conv, pf_ple_hist, pf_add_sum,
// pf_silu_bf16 and pf_to_bf16 (kernels/prefill_glue.hip:343-423, 552-566) and pf_hc_avg (kernels/prefill_attn.hip:388-397).
//
// The reference compiles these with contraction off: a sum of products here is a multiply and an add, never an fma, except
// where its source writes fmaf. Row sums follow the 256-thread tree of the other norms (thread t owns elements t, t + 256,
// ..; xor 16 .. 1 inside each group of 32 threads; the eight group sums in order).
#include "common.cuh"

#define GRID_1D(n4) dim3((unsigned)((((n4) + 255) / 256) < 1048576 ? (((n4) + 255) / 256) : 1048576))

// ---- gated RMSNorm of a GDN value head: y = ((o * rsqrt(mean(o^2) + eps)) * w) * (SILU ? silu(z) : sigmoid(z)) ------------
// silu for fp16 outputs (both kernels below, so a row's bits do not depend on the batch it came in): v_exp / v_rcp, rounded to 16 bits at once
CAMX_DEV float silu_fast16(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.442695041f)); }

// one wave per (token, head) row of K values (K % 4 == 0, K <= 1024); lane p holds elements 256 j + 4 p + k
template <bool SILU, bool F16OUT, int NI>
__global__ void __launch_bounds__(256) gdn_norm_rows(const float * __restrict__ o, const float * __restrict__ w, const float * __restrict__ z,
                                                     void * __restrict__ y, int K, float eps, long rows) {
    const int lane = slot_of(threadIdx.x & 63);
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    f32x4 ov[NI], zv[NI], wv[NI];
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int i0 = 256 * j + 4 * lane;
        ov[j] = zv[j] = wv[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        if (i0 < K) {
            ov[j] = __builtin_nontemporal_load((const f32x4 *)(o + row * K + i0));
            zv[j] = __builtin_nontemporal_load((const f32x4 *)(z + row * K + i0));
            wv[j] = *(const f32x4 *)(w + i0);
        }
    }
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < NI; j++) {                             // ss += o * o: a product, then a sum
        ss.x = ss.x + ov[j].x * ov[j].x; ss.y = ss.y + ov[j].y * ov[j].y; ss.z = ss.z + ov[j].z * ov[j].z; ss.w = ss.w + ov[j].w * ov[j].w;
    }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)K + eps);
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int i0 = 256 * j + 4 * lane;
        if (i0 < K) {
            f32x4 r;
#define G_(e) { const float nrm = (scale * ov[j].e) * wv[j].e; \
              r.e = F16OUT ? nrm * silu_fast16(zv[j].e) : (SILU ? nrm * (zv[j].e / (1.0f + expf(-zv[j].e))) : nrm * (1.0f / (1.0f + expf(-zv[j].e)))); }
            G_(x) G_(y) G_(z) G_(w)
#undef G_
            if (F16OUT) *(u32x2 *)((uint16_t *)y + row * K + i0) = pack_f16x4(r); else *(f32x4 *)((float *)y + row * K + i0) = r;
        }
    }
}

// K = 128 (the GDN value heads) at prefill sizes: a half-wave per row, two rows per wave instruction, U rows per half-wave
// with all their loads issued first. The logical threads past 128 hold zeros in the tree, so the four group sums of the row
// added in order are the whole sum. FAST (fp16 output only): silu from v_exp / v_rcp, rounded to 16 bits at once.
template <bool SILU, bool F16OUT, int U>
__global__ void __launch_bounds__(256) gdn_norm_128(const float * __restrict__ o, const float * __restrict__ w, const float * __restrict__ z,
                                                    void * __restrict__ y, float eps, long rows) {
    const int lane = slot_of(threadIdx.x & 63), l = lane & 31;
    const long span = (long)gridDim.x * 8;
    const long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
    f32x4 ov[U], zv[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const long r = r0 + u * span, rc = r < rows ? r : 0;
        ov[u] = __builtin_nontemporal_load((const f32x4 *)(o + rc * 128 + 4 * l));
        zv[u] = __builtin_nontemporal_load((const f32x4 *)(z + rc * 128 + 4 * l));
    }
    const f32x4 wv = *(const f32x4 *)(w + 4 * l);
#pragma unroll
    for (int u = 0; u < U; u++) {
        const long r = r0 + u * span;
        f32x4 ss;
        ss.x = 0.0f + ov[u].x * ov[u].x; ss.y = 0.0f + ov[u].y * ov[u].y; ss.z = 0.0f + ov[u].z * ov[u].z; ss.w = 0.0f + ov[u].w * ov[u].w;
        const float tot = half_groups_in_order<4>(group32_sum(ss), lane & 32);
        const float scale = rsqrt_exact(tot / 128.0f + eps);
        f32x4 rr;
#define G_(e) { const float nrm = (scale * ov[u].e) * wv.e; const float zz = zv[u].e; \
                rr.e = F16OUT ? nrm * silu_fast16(zz) : (SILU ? nrm * (zz / (1.0f + expf(-zz))) : nrm * (1.0f / (1.0f + expf(-zz)))); }
        G_(x) G_(y) G_(z) G_(w)
#undef G_
        if (r < rows) {
            if (F16OUT) __builtin_nontemporal_store(pack_f16x4(rr), (u32x2 *)((uint16_t *)y + r * 128 + 4 * l));
            else __builtin_nontemporal_store(rr, (f32x4 *)((float *)y + r * 128 + 4 * l));
        }
    }
}

// ---- GDN gates: gate = softplus(alpha + dt) * a, beta_sig = sigmoid(beta); y [T][2H] = gate | beta_sig -----------------------
__global__ void __launch_bounds__(256) gdn_gates_k(const float * __restrict__ al, int lda, const float * __restrict__ be, int ldb,
                                                   const float * __restrict__ dt, const float * __restrict__ A, float * __restrict__ y, int H, int T) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (q >= (long)T * H) return;
    const int tt = (int)(q / H), h = (int)(q - (long)tt * H);
    const float ab = al[(size_t)tt * lda + h] + dt[h];
    const float sp = ab > 20.0f ? ab : logf(1.0f + expf(ab));
    y[(size_t)tt * 2 * H + h] = sp * A[h];
    y[(size_t)tt * 2 * H + H + h] = 1.0f / (1.0f + expf(-be[(size_t)tt * ldb + h]));
}

// ---- fp16 KV append: cache[pos0 + t] = fp16(k[t]) | fp16(v[t]) -----------------------------------------------------------------
__global__ void __launch_bounds__(256) kv_append16_k(const float * __restrict__ k, int ldk, const float * __restrict__ v, int ldv,
                                                     uint16_t * __restrict__ cache, int M, int pos0, int rows, int * __restrict__ err, int vec,
                                                     const int32_t * __restrict__ posb) {
    if (posb) pos0 = posb[0];                             // the tape's device-resident position
    const int tt = blockIdx.x;
    const long pos = (long)pos0 + tt;
    if (pos < 0 || pos >= rows) { if (threadIdx.x == 0) atomicOr(err, 1); return; }
    uint16_t * c = cache + (size_t)pos * 2 * M;
    if (vec) {
        for (int i = 4 * threadIdx.x; i < M; i += 1024) {
            const f32x4 kv = __builtin_nontemporal_load((const f32x4 *)(k + (size_t)tt * ldk + i)), vv = __builtin_nontemporal_load((const f32x4 *)(v + (size_t)tt * ldv + i));
            __builtin_nontemporal_store(pack_f16x4(kv), (u32x2 *)(c + i)); __builtin_nontemporal_store(pack_f16x4(vv), (u32x2 *)(c + M + i));
        }
    } else {
        for (int i = threadIdx.x; i < M; i += 256) { c[i] = f2h_bits(k[(size_t)tt * ldk + i]); c[M + i] = f2h_bits(v[(size_t)tt * ldv + i]); }
    }
}

// ---- y = y + (a + b) ------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) add_sum_k(const float * __restrict__ a, const float * __restrict__ b, float * __restrict__ y, long n, int vec) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        if (q * 4 >= n) return;
        const f32x4 av = __builtin_nontemporal_load((const f32x4 *)a + q), bv = __builtin_nontemporal_load((const f32x4 *)b + q), yv = __builtin_nontemporal_load((const f32x4 *)y + q);
        f32x4 r; r.x = yv.x + (av.x + bv.x); r.y = yv.y + (av.y + bv.y); r.z = yv.z + (av.z + bv.z); r.w = yv.w + (av.w + bv.w);
        __builtin_nontemporal_store(r, (f32x4 *)y + q);
    } else {
        for (long i = q; i < n; i += (long)gridDim.x * 256) y[i] = y[i] + (a[i] + b[i]);
    }
}

// ---- the decode tape's remaining elementwise ops -------------------------------------------------------------------------------
// OP_OWN_F16 (kernels/k3_own_ops.h:247-252): y16 = fp16(x), round to nearest even
__global__ void __launch_bounds__(256) own_f16_k(const float * __restrict__ x, uint16_t * __restrict__ y, long n, int vec) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        if (q * 4 >= n) return;
        __builtin_nontemporal_store(pack_f16x4(__builtin_nontemporal_load((const f32x4 *)x + q)), (u32x2 *)y + q);
    } else {
        for (long i = q; i < n; i += (long)gridDim.x * 256) y[i] = f2h_bits(x[i]);
    }
}
// OP_OWN_MOE_SUM (kernels/k3_own_ops.h:255-256, 263-271): x[i] += acc, acc = 0 then, slot by slot, fma(w[s], d[s][i], acc) or (w null) acc + d[s][i]
__global__ void __launch_bounds__(256) own_moe_sum_k(const float * __restrict__ d, const float * __restrict__ w, float * __restrict__ x, long n, int S, int vec) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        if (q * 4 >= n) return;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int s = 0; s < S; s++) {
            const f32x4 dv = __builtin_nontemporal_load((const f32x4 *)(d + (size_t)s * n) + q);
            if (w) { const float ws = w[s]; acc.x = __builtin_fmaf(ws, dv.x, acc.x); acc.y = __builtin_fmaf(ws, dv.y, acc.y); acc.z = __builtin_fmaf(ws, dv.z, acc.z); acc.w = __builtin_fmaf(ws, dv.w, acc.w); }
            else { acc.x = acc.x + dv.x; acc.y = acc.y + dv.y; acc.z = acc.z + dv.z; acc.w = acc.w + dv.w; }
        }
        f32x4 xv = __builtin_nontemporal_load((const f32x4 *)x + q);
        xv.x += acc.x; xv.y += acc.y; xv.z += acc.z; xv.w += acc.w;
        __builtin_nontemporal_store(xv, (f32x4 *)x + q);
    } else {
        for (long i = q; i < n; i += (long)gridDim.x * 256) {
            float acc = 0.0f;
            for (int s = 0; s < S; s++) acc = w ? __builtin_fmaf(w[s], d[(size_t)s * n + i], acc) : acc + d[(size_t)s * n + i];
            x[i] += acc;
        }
    }
}
// OP_SHEXP_ADD (kernels/k3_gguf_ops.h:1218-1229): out[i] = moe[i] + shexp[i] * sigmoid(logit[token of i]), each step rounded on its own
__global__ void __launch_bounds__(256) shexp_add_k(const float * __restrict__ moe, const float * __restrict__ sh, const float * __restrict__ logit,
                                                   float * __restrict__ out, long n, int dd) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const float s = 1.0f / (1.0f + expf(-logit[i / dd]));
        const float g = sh[i] * s;
        out[i] = moe[i] + g;
    }
}
// rows of a multiple of 4 values, 16-byte aligned: the token in blockIdx.y, four values per lane, the gate once per lane
__global__ void __launch_bounds__(256) shexp_add_rows(const float * __restrict__ moe, const float * __restrict__ sh, const float * __restrict__ logit,
                                                      float * __restrict__ out, int dd4) {
    const int q = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    if (q >= dd4) return;
    const size_t e = (size_t)t * dd4 + q;
    const f32x4 m = __builtin_nontemporal_load((const f32x4 *)moe + e), h = __builtin_nontemporal_load((const f32x4 *)sh + e);
    const float s = 1.0f / (1.0f + expf(-logit[t]));
    f32x4 r;
    { const float g = h.x * s; r.x = m.x + g; } { const float g = h.y * s; r.y = m.y + g; }
    { const float g = h.z * s; r.z = m.z + g; } { const float g = h.w * s; r.w = m.w + g; }
    __builtin_nontemporal_store(r, (f32x4 *)out + e);
}

// ---- bf16 operand copies with zero rows up to Tpad: y[t][j] = bf16(SILU ? silu(fma(rs, x, 0)) : x) ---------------------------
// eight values per thread (K % 8 == 0, aligned): two 128-bit loads, one 128-bit non-temporal store
template <bool SILU>
__global__ void __launch_bounds__(256) to_bf16_rows8(const float * __restrict__ x, int ldx, uint16_t * __restrict__ y, int T, int Tpad, int K, float rs) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x, i = q * 8;
    if (i >= (long)Tpad * K) return;
    const int t = (int)(i / K), j = (int)(i - (long)t * K);
    u32x4 out = {0u, 0u, 0u, 0u};
    if (t < T) {
        f32x4 a = __builtin_nontemporal_load((const f32x4 *)(x + (size_t)t * ldx + j)), b = __builtin_nontemporal_load((const f32x4 *)(x + (size_t)t * ldx + j + 4));
        if (SILU) {
#define S_(v) { const float s = __builtin_fmaf(rs, v, 0.0f); v = s / (1.0f + expf(-s)); }
            S_(a.x) S_(a.y) S_(a.z) S_(a.w) S_(b.x) S_(b.y) S_(b.z) S_(b.w)
#undef S_
        }
        const u32x2 lo = pack_bf16x4_rne(a), hi = pack_bf16x4_rne(b);
        out = (u32x4){lo.x, lo.y, hi.x, hi.y};
    }
    __builtin_nontemporal_store(out, (u32x4 *)(y + i));
}
template <bool SILU>
__global__ void __launch_bounds__(256) to_bf16_rows(const float * __restrict__ x, int ldx, uint16_t * __restrict__ y, int T, int Tpad, int K, float rs, int vec) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    const int VW = vec ? 4 : 1;
    const long i = q * VW;
    if (i >= (long)Tpad * K) return;
    const int t = (int)(i / K), j = (int)(i - (long)t * K);
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (t < T) {
        if (vec) { const f32x4 xv = __builtin_nontemporal_load((const f32x4 *)(x + (size_t)t * ldx + j)); v[0] = xv.x; v[1] = xv.y; v[2] = xv.z; v[3] = xv.w; }
        else v[0] = x[(size_t)t * ldx + j];
        if (SILU) {
#pragma unroll
            for (int k = 0; k < 4; k++) { const float s = __builtin_fmaf(rs, v[k], 0.0f); v[k] = s / (1.0f + expf(-s)); }
        }
    }
    if (vec) *(u32x2 *)(y + i) = t < T ? pack_bf16x4_rne((f32x4){v[0], v[1], v[2], v[3]}) : (u32x2){0u, 0u};
    else y[i] = t < T ? to_bf16(v[0]) : (uint16_t)0;
}

// ---- hyper-connection average: y[t][i] = (((r0 + r1) + r2) + ..) * (1 / hc) of r [T][hc][D], y rows at ldo -------------------
__global__ void __launch_bounds__(256) hc_avg_k(const float * __restrict__ r, float * __restrict__ y, int T, int hc, int D, int ldo, int vec) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    const int VW = vec ? 4 : 1;
    const long i = q * VW;
    if (i >= (long)T * D) return;
    const int tt = (int)(i / D), ii = (int)(i - (long)tt * D);
    const float inv = 1.0f / (float)hc;
    if (vec) {
        f32x4 acc = __builtin_nontemporal_load((const f32x4 *)(r + (size_t)(tt * hc) * D + ii));
        for (int h = 1; h < hc; h++) acc = acc + __builtin_nontemporal_load((const f32x4 *)(r + (size_t)(tt * hc + h) * D + ii));
        acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
        if (vec == 2) __builtin_nontemporal_store(acc, (f32x4 *)(y + (size_t)tt * ldo + ii)); else *(f32x4 *)(y + (size_t)tt * ldo + ii) = acc;     // (2: a batch that streams from HBM)
    } else {
        float acc = r[(size_t)(tt * hc) * D + ii];
        for (int h = 1; h < hc; h++) acc = acc + r[(size_t)(tt * hc + h) * D + ii];
        y[(size_t)tt * ldo + ii] = acc * inv;
    }
}

// ---- per-layer-embedding gate: per token and stream st, s = (kn . qn) / sqrt(D), gate = sigmoid(sgn(s) sqrt(max(|s|, 1e-6))),
// gated[t][st][i] = val[t][i] * gate. qn given, or recomputed from the residual as (q * qscl[t * HC + st]) * qw[st][i].
// One workgroup per token; the dot product is the 256-thread tree with a product and a sum per element; HC <= 8.
__global__ void __launch_bounds__(256) ple_gate_k(const float * kn, const float * q, const float * qscl, const float * qw, const float * val, int ldv,
                                                  float * gated, float * gate_out, int HC, int D) {
    __shared__ float part[8][8];                         // [stream][half-wave]
    __shared__ float gate[8];
    const int tid = threadIdx.x, t = slot_of(tid), tt = blockIdx.x;
    const float * k_ = kn + (size_t)tt * HC * D, * q_ = q + (size_t)tt * HC * D, * v_ = val + (size_t)tt * ldv;
    // the streams' dot products side by side (each under its own 256-thread tree), one pair of barriers for all of them, and the
    // gates of the HC streams on HC threads
#pragma unroll
    for (int st = 0; st < 8; st++) {
        if (st < HC) {
            float acc = 0.0f;
            for (int i = t; i < D; i += 256) {
                const float qv = qscl ? (q_[(size_t)st * D + i] * qscl[tt * HC + st]) * qw[(size_t)st * D + i] : q_[(size_t)st * D + i];
                acc = acc + k_[(size_t)st * D + i] * qv;
            }
            acc += lane_xor16(acc); acc += lane_xor8(acc); acc += lane_xor4(acc); acc += lane_xor2(acc); acc += lane_xor1(acc);
            if ((tid & 31) == 0) part[st][tid >> 5] = acc;
        }
    }
    __syncthreads();
    if (tid < HC) {
        float sum = 0.0f;
        for (int w = 0; w < 8; w++) sum += part[tid][w];
        const float s = sum * (1.0f / sqrtf((float)D));
        const float mag = sqrtf(fmaxf(fabsf(s), 1e-6f));
        const float sgn = s > 0.0f ? 1.0f : (s < 0.0f ? -1.0f : 0.0f);
        const float gv = 1.0f / (1.0f + expf(-(sgn * mag)));
        gate[tid] = gv; gate_out[tt * HC + tid] = gv;
    }
    __syncthreads();
    // (gated may alias kn: every read of this token's kn rows is behind the barriers above)
    for (int c = tid; c < HC * D; c += 256) gated[(size_t)tt * HC * D + c] = v_[c % D] * gate[c / D];
}

// ---- per-layer-embedding conv: taps at t - 3 dil, t - 2 dil, t - dil, t with fp16 weights, every product and sum rounded
// separately, silu; inputs before the chunk from hist[c] = [x(-3 dil) .. x(-1)]; x given or recomputed as (x * xscl) * xw.
// y (optional) = conv; res (optional): res = res + (a + conv).
CAMX_DEV float ple_x(const float * x, const float * xscl, const float * xw, int tb, int c, int C, int D) {
    return xscl ? (x[(size_t)tb * C + c] * xscl[tb * (C / D) + c / D]) * xw[c] : x[(size_t)tb * C + c];
}
__global__ void __launch_bounds__(256) ple_conv_k(const float * __restrict__ x, const float * __restrict__ xscl, const float * __restrict__ xw,
                                                  const uint16_t * __restrict__ w, const float * __restrict__ hist, float * __restrict__ y,
                                                  const float * __restrict__ a, float * __restrict__ res, int C, int T, int D, int dil) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)T * C) return;
    const int t = (int)(i / C), c = (int)(i - (long)t * C), hl = 3 * dil;
    float conv = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int back = (3 - k) * dil;
        const float xv = back <= t ? ple_x(x, xscl, xw, t - back, c, C, D) : hist[(size_t)c * hl + hl - (back - t)];
        const float term = xv * h2f_bits(w[(size_t)c * 4 + k]);
        conv = k == 0 ? term : conv + term;
    }
    const float o = conv / (1.0f + expf(-conv));
    if (y) y[i] = o;
    if (res) { const float ab = a[i] + o; res[i] = res[i] + ab; }
}
// the same for C % 4 == 0, D % 4 == 0 and 16-byte aligned operands: the token in blockIdx.y (no division of an element index), four
// channels per thread (their sixteen fp16 weights in two 16-byte loads), streamed outputs non-temporal
__global__ void __launch_bounds__(256) ple_conv_rows(const float * __restrict__ x, const float * __restrict__ xscl, const float * __restrict__ xw,
                                                     const uint16_t * __restrict__ w, const float * __restrict__ hist, float * __restrict__ y,
                                                     const float * __restrict__ a, float * __restrict__ res, int C, int D, int dil) {
    // workgroup i runs on XCD i mod 8, each with its own L2: an XCD takes a contiguous range of tokens, so that the three earlier rows a
    // token reads were fetched into the same L2 by its neighbours a moment ago (with tokens dealt round-robin every row crossed the fabric
    // four times: 67 MB read for 17 MB of input at 4096 x 1024)
    int t = blockIdx.y, bx = blockIdx.x;
    const int total = gridDim.x * gridDim.y;
    if ((total & 7) == 0) {
        const int lin = blockIdx.x + gridDim.x * blockIdx.y, nw = (lin & 7) * (total >> 3) + (lin >> 3);
        t = nw / gridDim.x; bx = nw - t * gridDim.x;
    }
    const int c = 4 * (bx * 256 + threadIdx.x), hl = 3 * dil;
    if (c >= C) return;
    const u32x4 w0 = *(const u32x4 *)(w + (size_t)c * 4), w1 = *(const u32x4 *)(w + (size_t)c * 4 + 8);
    const uint32_t ww[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};      // channel j's taps: halves 4 j .. 4 j + 3
    f32x4 xwv = {1.0f, 1.0f, 1.0f, 1.0f};
    if (xscl) xwv = *(const f32x4 *)(xw + c);
    float conv[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int back = (3 - k) * dil;
        float xv[4];
        if (back <= t) {
            const int tb = t - back;
            const f32x4 v = *(const f32x4 *)(x + (size_t)tb * C + c);
            xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
            if (xscl) {
                const float sc = xscl[tb * (C / D) + c / D];
                xv[0] = (xv[0] * sc) * xwv.x; xv[1] = (xv[1] * sc) * xwv.y; xv[2] = (xv[2] * sc) * xwv.z; xv[3] = (xv[3] * sc) * xwv.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) xv[j] = hist[(size_t)(c + j) * hl + hl - (back - t)];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t pair = ww[2 * j + (k >> 1)];
            const float term = xv[j] * h2f_bits((uint16_t)((k & 1) ? pair >> 16 : pair & 0xffffu));
            conv[j] = k == 0 ? term : conv[j] + term;
        }
    }
    f32x4 o;
    o.x = conv[0] / (1.0f + expf(-conv[0])); o.y = conv[1] / (1.0f + expf(-conv[1]));
    o.z = conv[2] / (1.0f + expf(-conv[2])); o.w = conv[3] / (1.0f + expf(-conv[3]));
    const size_t i = (size_t)t * C + c;
    if (y) __builtin_nontemporal_store(o, (f32x4 *)(y + i));
    if (res) {
        const f32x4 av = __builtin_nontemporal_load((const f32x4 *)(a + i)), rv = __builtin_nontemporal_load((const f32x4 *)(res + i));
        f32x4 r; r.x = rv.x + (av.x + o.x); r.y = rv.y + (av.y + o.y); r.z = rv.z + (av.z + o.z); r.w = rv.w + (av.w + o.w);
        __builtin_nontemporal_store(r, (f32x4 *)(res + i));
    }
}
// hist[c] = the last 3 dil inputs of [hist[c], x[0 .. T - 1][c]]; 3 dil <= 32
__global__ void __launch_bounds__(256) ple_hist_k(const float * __restrict__ x, const float * __restrict__ xscl, const float * __restrict__ xw,
                                                  float * __restrict__ hist, int C, int T, int D, int dil) {
    const int c = blockIdx.x * 256 + threadIdx.x, hl = 3 * dil;
    if (c >= C) return;
    float h[32];
#pragma unroll
    for (int j = 0; j < 32; j++) {
        h[j] = 0.0f;
        if (j < hl) { const int tj = T - hl + j; h[j] = tj < 0 ? hist[(size_t)c * hl + hl + tj] : ple_x(x, xscl, xw, tj, c, C, D); }
    }
#pragma unroll
    for (int j = 0; j < 32; j++) if (j < hl) hist[(size_t)c * hl + j] = h[j];
}

extern "C" {

// pf_gdn_norm (silu = 0: sigmoid gate; 1: silu gate, the reference's PF_GDN_SILU build) and q35p_gdn_norm16 (f16 = 1, silu gate)
static int gdn_norm_launch(const float * o, const float * w, const float * z, void * y, int K, float eps, long rows, int silu, int f16, hipStream_t st) {
    if (!o || !w || !z || !y || K < 4 || K % 4 || K > 1024 || rows < 0 || (((uintptr_t)o | (uintptr_t)w | (uintptr_t)z) & 15) || ((uintptr_t)y & (f16 ? 7 : 15)))
        return CAMX_EINVAL;
    if (rows == 0) return CAMX_OK;
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (K == 128 && rows >= 32768) {                                     // a prefill chunk: four rows per half-wave
        const dim3 g4((unsigned)((rows + 31) / 32));
        if (f16) gdn_norm_128<true, true, 4><<<g4, block, 0, st>>>(o, w, z, y, eps, rows);
        else if (silu) gdn_norm_128<true, false, 4><<<g4, block, 0, st>>>(o, w, z, y, eps, rows);
        else gdn_norm_128<false, false, 4><<<g4, block, 0, st>>>(o, w, z, y, eps, rows);
        CAMX_LAUNCH_RET();
    }
    const int ni = (K + 255) / 256;
#define GN(S, F, N) gdn_norm_rows<S, F, N><<<grid, block, 0, st>>>(o, w, z, y, K, eps, rows)
#define GN_NI(S, F) { if (ni == 1) GN(S, F, 1); else if (ni == 2) GN(S, F, 2); else GN(S, F, 4); }
    if (f16) GN_NI(true, true) else if (silu) GN_NI(true, false) else GN_NI(false, false)
#undef GN_NI
#undef GN
    CAMX_LAUNCH_RET();
}
int camx_pf_gdn_norm(const float * o, const float * w, const float * z, float * y, int K, float eps, long rows, int silu, hipStream_t st) {
    return gdn_norm_launch(o, w, z, y, K, eps, rows, silu, 0, st);
}
int camx_q35p_gdn_norm16(const float * o, const float * w, const float * z, uint16_t * y16, int K, float eps, long rows, hipStream_t st) {
    return gdn_norm_launch(o, w, z, y16, K, eps, rows, 1, 1, st);
}
int camx_pf_gdn_gates(const float * al, int lda, const float * be, int ldb, const float * dt, const float * A, float * y, int H, int T, hipStream_t st) {
    if (!al || !be || !dt || !A || !y || H < 1 || T < 0 || lda < H || ldb < H) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if ((long)T * H >= 0x7fffffffL * 256) return CAMX_EINVAL;
    gdn_gates_k<<<dim3((unsigned)(((long)T * H + 255) / 256)), dim3(256), 0, st>>>(al, lda, be, ldb, dt, A, y, H, T);
    CAMX_LAUNCH_RET();
}
// (internal: also the fp16 form of camx_op_kv_append, whose position is a device word)
int camx_i_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, const int32_t * posb, int rows, int * err, int T, hipStream_t st) {
    if (!k || !v || !cache || !err || M < 1 || ldk < M || ldv < M || T < 0 || ((uintptr_t)cache & 1)) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const int vec = !((M | ldk | ldv) & 3) && !(((uintptr_t)k | (uintptr_t)v) & 15) && !((uintptr_t)cache & 7);
    kv_append16_k<<<dim3(T), dim3(256), 0, st>>>(k, ldk, v, ldv, cache, M, pos0, rows, err, vec, posb);
    CAMX_LAUNCH_RET();
}
int camx_q35p_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, int rows, int * err, int T, hipStream_t st) {
    return camx_i_kv_append16(k, ldk, v, ldv, cache, M, pos0, nullptr, rows, err, T, st);
}
int camx_pf_add_sum(const float * a, const float * b, float * y, long n, hipStream_t st) {
    if (!a || !b || !y || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int vec = n % 4 == 0 && !(((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15) && n / 4 < 0x7fffffffL * 256;
    add_sum_k<<<vec ? dim3((unsigned)((n / 4 + 255) / 256)) : GRID_1D(n), dim3(256), 0, st>>>(a, b, y, n, vec);
    CAMX_LAUNCH_RET();
}
int camx_gg_quantize_q8_1(const float * x, void * y, long n, int mode, float rs, const float * g, hipStream_t st);                 // quant.hip
int camx_gate_mul(const void * a, const void * gate, void * y, long N, int D, int stride, int off, int io, hipStream_t st);         // elt.hip
// The decode tape's ops next to the ones above, by their Seg fields (python/caminus/engine/k3.py): the same arithmetic as the prefill kernels
// of the same names, which the reference states in both places (kernels/k3_gguf_ops.h:1356-1372, 1461-1489, 1607-1619, 1683-1692;
// kernels/k3_q35_ops.h:196-211, 314-333).
// OP_ADD_SUM (k3.py:1237-1242): a, W = b, y in place, N = n
int camx_op_add_sum(const float * a, const float * b, float * y, int n, hipStream_t st) { return camx_pf_add_sum(a, b, y, (long)n, st); }
// OP_GDN_GATES (k3.py:1010-1015): a = alpha [T][H], W = beta [T][H], gs = dt [H], asum = ssm_a [H], y = out [T][2H], N = H
int camx_op_gdn_gates(const float * alpha, const float * beta, const float * dt, const float * a, float * out, int H, int T, hipStream_t st) {
    return camx_pf_gdn_gates(alpha, H, beta, H, dt, a, out, H, T, st);
}
// OP_GDN_NORM (k3.py:1037-1043): a = o [N][K], W = w [K], gs = z, y = out, asum = q8 (optional: q8_1 blocks of out, K % 32 == 0), rs = eps,
// N = T * H heads, K = S; silu: the K3_GDN_SILU builds (silu(z) instead of sigmoid(z))
int camx_op_gdn_norm(const float * o, const float * w, const float * z, float * out, void * q8, int N, int K, float eps, int silu, hipStream_t st) {
    if (N < 0 || silu < 0 || silu > 1 || (q8 && (K & 31))) return CAMX_EINVAL;
    const int rc = camx_pf_gdn_norm(o, w, z, out, K, eps, (long)N, silu, st);
    if (rc || !q8 || N == 0) return rc;
    return camx_gg_quantize_q8_1(out, q8, (long)N * K, 0, 0.0f, nullptr, st);      // q8_emit of every stored value (kernels/k3_gguf_ops.h:1486)
}
// OP_GDN_NORM16 (k3.py:1045-1055): the SiLU form, y = out16 fp16
int camx_op_gdn_norm16(const float * o, const float * w, const float * z, uint16_t * out16, int N, int K, float eps, hipStream_t st) {
    return N < 0 ? CAMX_EINVAL : camx_q35p_gdn_norm16(o, w, z, out16, K, eps, (long)N, st);
}
// OP_GATE_MUL (k3.py:1201-1207): a, W = gate, y = out fp32, asum = q8 (optional, n % 32 == 0), N = n, K = dim, pad1 = head_stride, pad2 = offset
int camx_op_gate_mul(const float * a, const float * gate, int head_stride, int offset, float * out, void * q8, int n, int dim, hipStream_t st) {
    if (n < 0 || (q8 && (n & 31))) return CAMX_EINVAL;
    const int rc = camx_gate_mul(a, gate, out, (long)n, dim, head_stride, offset, 0, st);
    if (rc || !q8 || n == 0) return rc;
    return camx_gg_quantize_q8_1(out, q8, (long)n, 0, 0.0f, nullptr, st);
}
// OP_OWN_F16 (k3.py:846-852): a = x, y = out fp16, N = n
int camx_op_own_f16(const float * x, uint16_t * out16, int n, hipStream_t st) {
    if (!x || !out16 || n < 0) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int vec = n % 4 == 0 && !((uintptr_t)x & 15) && !((uintptr_t)out16 & 7);
    own_f16_k<<<vec ? dim3((unsigned)((n / 4 + 255) / 256)) : GRID_1D(n), dim3(256), 0, st>>>(x, out16, n, vec);
    CAMX_LAUNCH_RET();
}
// OP_OWN_MOE_SUM (k3.py:862-868): a = d [slots][n], gs = w [slots] or null (weights 1), y = x in place, N = n, pad1 = slots (1 .. 64)
int camx_op_own_moe_sum(const float * d, const float * w, float * x, int n, int slots, hipStream_t st) {
    if (!d || !x || n < 0 || slots < 1 || slots > 64) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int vec = n % 4 == 0 && !(((uintptr_t)d | (uintptr_t)x) & 15);
    own_moe_sum_k<<<vec ? dim3((unsigned)((n / 4 + 255) / 256)) : GRID_1D(n), dim3(256), 0, st>>>(d, w, x, n, slots, vec);
    CAMX_LAUNCH_RET();
}
// OP_SHEXP_ADD (k3.py:958-963): a = moe, W = shexp, gs = gate logit [T], y = out, N = n (T tokens of n / T values)
int camx_op_shexp_add(const float * moe, const float * shexp, const float * gate_logit, float * out, int n, int T, hipStream_t st) {
    if (!moe || !shexp || !gate_logit || !out || n < 0 || T < 1 || n % T) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const int dd = n / T;
    if (dd % 4 == 0 && T <= 65535 && !(((uintptr_t)moe | (uintptr_t)shexp | (uintptr_t)out) & 15))
        shexp_add_rows<<<dim3((unsigned)((dd / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st>>>(moe, shexp, gate_logit, out, dd / 4);
    else shexp_add_k<<<GRID_1D(n), dim3(256), 0, st>>>(moe, shexp, gate_logit, out, n, dd);
    CAMX_LAUNCH_RET();
}
static int to_bf16_launch(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, float rs, bool silu, hipStream_t st) {
    if (!x || !y || T < 0 || Tpad < T || K < 1 || ldx < K) return CAMX_EINVAL;
    if (Tpad == 0) return CAMX_OK;
    if (!((K | ldx) & 7) && !(((uintptr_t)x | (uintptr_t)y) & 15) && (long)Tpad * K / 8 < 0x7fffffffL * 256) {
        const dim3 g8((unsigned)(((long)Tpad * K / 8 + 255) / 256));
        if (silu) to_bf16_rows8<true><<<g8, dim3(256), 0, st>>>(x, ldx, y, T, Tpad, K, rs); else to_bf16_rows8<false><<<g8, dim3(256), 0, st>>>(x, ldx, y, T, Tpad, K, rs);
        CAMX_LAUNCH_RET();
    }
    const int vec = !((K | ldx) & 3) && !((uintptr_t)x & 15) && !((uintptr_t)y & 7);
    const long n = (long)Tpad * K / (vec ? 4 : 1);
    if (n >= 0x7fffffffL * 256) return CAMX_EINVAL;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (silu) to_bf16_rows<true><<<grid, block, 0, st>>>(x, ldx, y, T, Tpad, K, rs, vec); else to_bf16_rows<false><<<grid, block, 0, st>>>(x, ldx, y, T, Tpad, K, rs, vec);
    CAMX_LAUNCH_RET();
}
int camx_pf_silu_bf16(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, float rs, hipStream_t st) { return to_bf16_launch(x, ldx, y, T, Tpad, K, rs, true, st); }
int camx_pf_to_bf16(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, hipStream_t st) { return to_bf16_launch(x, ldx, y, T, Tpad, K, 0.0f, false, st); }
int camx_pf_hc_avg(const float * r, float * y, int T, int hc, int D, int ldo, hipStream_t st) {
    if (!r || !y || T < 0 || hc < 1 || D < 1 || ldo < D) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const int vec = !((D | ldo) & 3) && !(((uintptr_t)r | (uintptr_t)y) & 15) ? ((long)T * D >= (1L << 20) ? 2 : 1) : 0;
    const long n = (long)T * D / (vec ? 4 : 1);
    hc_avg_k<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(r, y, T, hc, D, ldo, vec);
    CAMX_LAUNCH_RET();
}
int camx_pf_ple_gate(const float * kn, const float * q, const float * qscl, const float * qw, const float * val, int ldv, float * gated, float * gate_out,
                     int HC, int D, int T, hipStream_t st) {
    if (!kn || !q || !val || !gated || !gate_out || HC < 1 || HC > 8 || D < 1 || ldv < D || T < 0 || ((qscl == nullptr) != (qw == nullptr))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    ple_gate_k<<<dim3(T), dim3(256), 0, st>>>(kn, q, qscl, qw, val, ldv, gated, gate_out, HC, D);
    CAMX_LAUNCH_RET();
}
int camx_pf_ple_conv(const float * x, const float * xscl, const float * xw, const uint16_t * w, const float * hist, float * y, const float * a, float * res,
                     int C, int T, int D, int dil, hipStream_t st) {
    if (!x || !w || !hist || (!y && !res) || (res && !a) || C < 1 || T < 0 || D < 1 || C % D || dil < 1 || ((xscl == nullptr) != (xw == nullptr))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if ((long)T * C >= 0x7fffffffL * 256) return CAMX_EINVAL;
    if (C % 4 == 0 && D % 4 == 0 && T <= 65535 && !(((uintptr_t)x | (uintptr_t)xw | (uintptr_t)w | (uintptr_t)y | (uintptr_t)a | (uintptr_t)res) & 15)) {
        ple_conv_rows<<<dim3((unsigned)((C / 4 + 255) / 256), (unsigned)T), dim3(256), 0, st>>>(x, xscl, xw, w, hist, y, a, res, C, D, dil);
        CAMX_LAUNCH_RET();
    }
    ple_conv_k<<<dim3((unsigned)(((long)T * C + 255) / 256)), dim3(256), 0, st>>>(x, xscl, xw, w, hist, y, a, res, C, T, D, dil);
    CAMX_LAUNCH_RET();
}
int camx_pf_ple_hist(const float * x, const float * xscl, const float * xw, float * hist, int C, int T, int D, int dil, hipStream_t st) {
    if (!x || !hist || C < 1 || T < 0 || D < 1 || C % D || dil < 1 || 3 * dil > 32 || ((xscl == nullptr) != (xw == nullptr))) return CAMX_EINVAL;
    ple_hist_k<<<dim3((unsigned)((C + 255) / 256)), dim3(256), 0, st>>>(x, xscl, xw, hist, C, T, D, dil);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
