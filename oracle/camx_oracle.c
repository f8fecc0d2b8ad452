/* CPU oracle for the fused per-layer row kernels: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's arithmetic, one function per kernel family, each citing the reference
 * file:line it follows (paths relative to the reference checkout). Only tests, the smoke check and the benchmark's
 * CPU-baseline leg may load this library; the product path never does.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC (see oracle/build.py). With contraction off the
 * compiler never fuses a*b+c; every fused multiply-add the reference states is written fmaf() here.
 *
 * Numeric classes. INT: bit-exact by construction (adds/subs/muls/divs/sqrt are IEEE, reduction trees are explicit).
 * FP: functions that call libm transcendentals (expf, cosf, sinf, powf) are compared with a tolerance, because the
 * reference's device libm, glibc and the gfx950 device libm round those differently.
 *
 * Contract decisions where the reference's device instruction cannot be restated on a CPU:
 *   rsqrtf(v)  -> 1.0f / sqrtf(v), both correctly rounded (the reference runs an approximate v_rsq_f32).
 *   sum trees  -> 256 logical threads, thread t owns elements t, t + 256, ...; an fmaf chain in element order; the
 *                 32-lane xor butterfly (16, 8, 4, 2, 1) inside each group of 32 threads; the 8 group sums added in
 *                 order from 0.0f (kernels/k3_own_ops.h:373-377, kernels/q35_prefill.hip:644-656).
 *
 * Pinned by (tests/test_oracle_*.py): the reference's literal Q8 KV byte vectors (tests/io/test_ref_kv.py:39-172), its
 * seeded block generator (tests/io/test_own_kv_codec.py:24-68), the compiled reference header own_kv_codec.h
 * (oracle/_ref), scalar per-value format definitions (tests/io/test_own_formats.py:31-68), the float64 Sylvester
 * Hadamard (tests/engine/test_q3moe_kvq8_cpu.py:153-173), the YaRN table expectations
 * (tests/engine/test_q3m_yarn_rope.py:57-62), q8_host (tests/engine/golden_util.py:101-110) and float64 closed forms.
 * orc_actq_* / orc_silu_mul_actq_* / orc_block_entry_* (forward and backward): the reference's own tests compare with torch
 * ops under bf16 autocast (tests/train/test_silu_mul_actq.py:29-37, tests/train/test_block_entry.py:17-33) through its
 * private trainer's fq_act, which is not in the tree; the same graph, written from the kernel file's statement of it
 * (kernels/actq.hip:1-12), is evaluated and differentiated by torch on the CPU in tests/test_oracle_actq_autograd.py.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* threads for the row loops (0: the runtime's default); returns the previous setting. Timing only: results do not depend on it */
ORC_API int orc_set_threads(int n) {
#ifdef _OPENMP
    const int before = omp_get_max_threads();
    omp_set_num_threads(n > 0 ? n : omp_get_num_procs());
    return before;
#else
    (void)n;
    return 1;
#endif
}

/* ---- conversions (kernels/core.hip:14-21, kernels/prefill_glue.hip:77-80) ------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

ORC_API float orc_bf2f(uint16_t h) { return u2f((uint32_t)h << 16); }

/* f2bf: round to nearest even, any NaN -> 0x7fc0 (kernels/core.hip:16-21) */
ORC_API uint16_t orc_f2bf(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
/* to_bf16: the same rounding without the NaN case (kernels/prefill_glue.hip:77-80) */
ORC_API uint16_t orc_to_bf16(float f) {
    const uint32_t u = f2u(f);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static inline float rbf(float f) { return orc_bf2f(orc_f2bf(f)); }

/* fp32 -> fp16 bits, round to nearest even, IEEE subnormals, overflow to inf ((_Float16)x) */
ORC_API uint16_t orc_f2h(float f) {
    const uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x1ffu));   /* NaN stays NaN (quiet) */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                           /* >= 65536 or inf */
    if (a >= 0x38800000u) {                                                            /* normal half range */
        const uint32_t m = a - 0x38000000u;                                            /* rebias exponent by 112 */
        uint32_t r = m >> 13;
        const uint32_t rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;                        /* may carry into inf: correct */
        return (uint16_t)(sign | r);
    }
    if (a < 0x33000000u) return (uint16_t)sign;                                        /* < 2^-25 -> 0 */
    /* subnormal half: value = mant * 2^(e-150), target unit 2^-24 */
    const int e = (int)(a >> 23);
    const uint32_t mant = (a & 0x7fffffu) | 0x800000u;
    const int sh = 126 - e;                                                            /* 14 .. 24 */
    uint32_t r = mant >> sh;
    const uint32_t rem = mant & ((1u << sh) - 1u), half = 1u << (sh - 1);
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}
ORC_API float orc_h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1fu) return u2f(sign | 0x7f800000u | (m << 13));
    if (e) return u2f(sign | ((e + 112u) << 23) | (m << 13));
    if (!m) return u2f(sign);
    const float v = (float)m * 0x1p-24f;                                               /* exact */
    return sign ? -v : v;
}
static inline float f16r(float x) { return orc_h2f(orc_f2h(x)); }                      /* kernels/own_kv_rot128.h:17-19 */

ORC_API void orc_f2h_n(const float * x, uint16_t * y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = orc_f2h(x[i]); }
ORC_API void orc_h2f_n(const uint16_t * x, float * y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = orc_h2f(x[i]); }

/* ---- reduction trees ------------------------------------------------------------------------------------------------- */
/* the 32-lane xor butterfly: v[l] += v[l ^ o] for o = 16, 8, 4, 2, 1 (kernels/own_quant.h:26-30, q3m_prefill.hip:351-355) */
static float bfly32_sum(const float * in) {
    float v[32], n[32];
    memcpy(v, in, sizeof v);
    for (int o = 16; o > 0; o >>= 1) {
        for (int l = 0; l < 32; l++) n[l] = v[l] + v[l ^ o];
        memcpy(v, n, sizeof v);
    }
    return v[0];
}
ORC_API float orc_bfly32_sum(const float * v) { return bfly32_sum(v); }

/* sum of squares of a row under the contract tree; threads = 256 (rows) or 128 (a 128-wide head: 4 groups) */
static float row_ss(const float * x, int n) {
    float part[256];
    for (int t = 0; t < 256; t++) part[t] = 0.0f;
    for (int i = 0; i < n; i++) part[i & 255] = fmaf(x[i], x[i], part[i & 255]);
    float tot = 0.0f;
    for (int g = 0; g < 8; g++) tot += bfly32_sum(part + 32 * g);
    return tot;
}
ORC_API float orc_row_ss(const float * x, int n) { return row_ss(x, n); }
static inline float rsqrt_c(float v) { return 1.0f / sqrtf(v); }

/* ---- q8_1 (36-byte ggml block): kernels/k3_gguf_ops.h:146-162, kernels/k3_gguf.hip:29-36 ---------------------------- */
static inline float silu_f(float x) { return x / (1.0f + expf(-x)); }                  /* k3_gguf_ops.h:53 */
/* (int8_t)roundf(v). In range (|v| <= 127: every block whose scale is a normal number) this is the C conversion. Out of range the
 * C conversion is undefined; the reference's kernels run it as the GPU's float -> int32 conversion, which saturates (NaN -> 0), and
 * then keep the low byte. That is what is stated here, so that blocks whose scale underflows (amax below 127 * FLT_TRUE_MIN for
 * q8_1, 127 / amax = inf for the MMQ layout) have defined bytes: +inf -> 0x7fffffff -> -1, -inf -> 0x80000000 -> 0. */
static inline int8_t roundf_i8(float v) {
    const float r = roundf(v);
    if (r != r) return 0;
    if (r >= 2147483648.0f) return (int8_t)0xff;
    if (r <= -2147483648.0f) return 0;
    return (int8_t)(uint8_t)((uint32_t)(int32_t)r & 0xffu);
}

static void q8_1_block(const float * xi, uint8_t * blk) {
    float amax = 0.0f;
    for (int l = 0; l < 32; l++) amax = fmaxf(amax, fabsf(xi[l]));
    const float sum = bfly32_sum(xi);
    const float d = amax / 127.0f;
    const uint16_t hd = orc_f2h(d), hs = orc_f2h(sum);
    memcpy(blk, &hd, 2); memcpy(blk + 2, &hs, 2);
    for (int l = 0; l < 32; l++) blk[4 + l] = (uint8_t)(amax == 0.0f ? 0 : roundf_i8(xi[l] / d));
}
/* mode 0 plain, 1 silu(x * rs), 2 silu(x) * g[i] (k3_gguf_ops.h:55-77); values past n quantize as 0 */
ORC_API void orc_q8_1(const float * x, uint8_t * y, int64_t n, int mode, float rs, const float * g) {
    const int64_t nb = (n + 31) / 32;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; b++) {
        float xi[32];
        for (int l = 0; l < 32; l++) {
            const int64_t i = b * 32 + l;
            float v = i < n ? x[i] : 0.0f;
            if (mode == 1 && i < n) { const float t = v * rs; v = silu_f(t); }
            if (mode == 2 && i < n) v = silu_f(v) * g[i];
            xi[l] = v;
        }
        q8_1_block(xi, y + b * 36);
    }
}

/* ---- q8_1 in the MMQ layout (144 bytes per 128 values): kernels/ggml_mmq/quantize_mmq.cuh:41-140 --------------------- */
/* layout 0 = D4 (fp32 d per 32 values), 1 = DS4 (half2(d, sum)). Column c of y is row (ids ? ids[c] : c) of x (row
 * stride s01 floats). K is padded with zeros to a multiple of 512. amax == 0: codes 0, d = 0, sum = 0 (the vendored
 * kernel computes 0 * inf there; the cast of that NaN is 0 on the reference's hardware). */
static void mmq_quant32(const float * v, int layout, uint8_t * blk, int sub) {
    float amax8[8], sum8[8];
    for (int t = 0; t < 8; t++) {
        const float * p = v + 4 * t;
        float a = fabsf(p[0]); a = fmaxf(a, fabsf(p[1])); a = fmaxf(a, fabsf(p[2])); a = fmaxf(a, fabsf(p[3]));
        amax8[t] = a;
        sum8[t] = ((p[0] + p[1]) + p[2]) + p[3];
    }
    float amax = 0.0f;
    for (int t = 0; t < 8; t++) amax = fmaxf(amax, amax8[t]);
    float s[8], n8[8];
    memcpy(s, sum8, sizeof s);
    for (int o = 4; o > 0; o >>= 1) { for (int t = 0; t < 8; t++) n8[t] = s[t] + s[t ^ o]; memcpy(s, n8, sizeof s); }
    float d;
    int8_t * qs = (int8_t *)(blk + 16 + 32 * sub);
    if (amax == 0.0f) { d = 0.0f; for (int l = 0; l < 32; l++) qs[l] = 0; }
    else {
        const float d_inv = 127.0f / amax;
        for (int l = 0; l < 32; l++) qs[l] = roundf_i8(v[l] * d_inv);
        d = 1.0f / d_inv;
    }
    if (layout == 1) { const uint16_t hd = orc_f2h(d), hs = orc_f2h(s[0]); memcpy(blk + 4 * sub, &hd, 2); memcpy(blk + 4 * sub + 2, &hs, 2); }
    else memcpy(blk + 4 * sub, &d, 4);
}
ORC_API void orc_mmq_q8_1(const float * x, const int32_t * ids, uint8_t * y, int64_t K, int64_t s01, int ncols, int layout) {
    const int64_t Kp = (K + 511) / 512 * 512, nkb = Kp / 128;
#pragma omp parallel for schedule(static)
    for (int c = 0; c < ncols; c++) {
        const float * xr = x + (int64_t)(ids ? ids[c] : c) * s01;
        for (int64_t kb = 0; kb < nkb; kb++) {
            uint8_t * blk = y + (kb * ncols + c) * 144;
            for (int sub = 0; sub < 4; sub++) {
                float v[32];
                for (int l = 0; l < 32; l++) { const int64_t i = kb * 128 + sub * 32 + l; v[l] = i < K ? xr[i] : 0.0f; }
                mmq_quant32(v, layout, blk, sub);
            }
        }
    }
}
/* scatter form: token t's row (stride s_tok) quantized once, written to columns ids_inv[t * k + slot] of ncols = ntok * k */
ORC_API void orc_mmq_q8_1_scatter(const float * x, const int32_t * ids_inv, uint8_t * y, int64_t K, int64_t s_tok, int ntok, int k, int layout) {
    const int64_t Kp = (K + 511) / 512 * 512, nkb = Kp / 128, ncols = (int64_t)ntok * k;
    for (int t = 0; t < ntok; t++) {
        const float * xr = x + (int64_t)t * s_tok;
        for (int64_t kb = 0; kb < nkb; kb++) {
            uint8_t tmp[144];
            for (int sub = 0; sub < 4; sub++) {
                float v[32];
                for (int l = 0; l < 32; l++) { const int64_t i = kb * 128 + sub * 32 + l; v[l] = i < K ? xr[i] : 0.0f; }
                mmq_quant32(v, layout, tmp, sub);
            }
            for (int slot = 0; slot < k; slot++) memcpy(y + (kb * ncols + ids_inv[(int64_t)t * k + slot]) * 144, tmp, 144);
        }
    }
}

/* ---- residual add + RMSNorm family --------------------------------------------------------------------------------- */
/* q3p_add_rms16 / OP_OWN_ADD_RMS16 (kernels/q3m_prefill.hip:385-415, kernels/k3_own_ops.h:326-383):
 *   x[i] += sum_s w[s] d[s][i] (fmaf in slot order from 0; w NULL: acc + d; S = 0: no add), x written back when S > 0;
 *   h = (x * scale) * nw, h16 = fp16(h). d [n][S][N], w [n][S]. h may be NULL. q8 (optional): the q8_1 copy of h. */
ORC_API void orc_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps,
                           float * h, uint16_t * h16, uint8_t * q8, int N, int n) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        float * xr = x + (size_t)t * N;
        const float * dr = d ? d + (size_t)t * S * N : NULL;
        const float * wr = w ? w + (size_t)t * S : NULL;
        if (S > 0)
            for (int i = 0; i < N; i++) {
                float acc = 0.0f;
                for (int s = 0; s < S; s++) acc = wr ? fmaf(wr[s], dr[(size_t)s * N + i], acc) : acc + dr[(size_t)s * N + i];
                xr[i] += acc;
            }
        const float scale = rsqrt_c(row_ss(xr, N) / (float)N + eps);
        float hv[32];
        for (int i = 0; i < N; i++) {
            const float v = (xr[i] * scale) * nw[i];
            if (h) h[(size_t)t * N + i] = v;
            if (h16) h16[(size_t)t * N + i] = orc_f2h(v);
            if (q8) { hv[i & 31] = v; if ((i & 31) == 31) q8_1_block(hv, q8 + ((size_t)t * N + i) / 32 * 36); }
        }
    }
}
/* q35p_add_rms16 (kernels/q35_prefill.hip:636-660): x = x + d directly (d NULL: no add), any N = 256 NI */
/* the product of two floats rounded ONCE to half: the product is exact in double (24 + 24 significant bits), the conversion below rounds it
 * to nearest even. This is what the reference's q35p_add_rms16 binary stores in h16: its compiler rounds the fp16 copy straight from the
 * last product (v_fma_mixlo_f16), and the reference keeps its source shaped so that it does (kernels/q35_prefill.hip:630-635). */
static uint16_t d2h(double v) {
    uint64_t u; memcpy(&u, &v, 8);
    const uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    const double a = fabs(v);
    if (a != a) return (uint16_t)(sign | 0x7e00u);
    if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);                 /* rounds to 2^16: infinity */
    if (a < 0x1p-14) return (uint16_t)(sign | (uint16_t)nearbyint(a * 0x1p24));       /* subnormal halves (and 2^-14 itself by carry) */
    int e; const double m = frexp(a, &e);                                 /* a = m 2^e, m in [0.5, 1) */
    uint32_t mant = (uint32_t)nearbyint(m * 2048.0);                      /* 11 bits, ties to even */
    if (mant == 2048u) { mant = 1024u; e++; }
    return (uint16_t)(sign | (uint32_t)((e - 1 + 15) << 10) | (mant - 1024u));
}
ORC_API uint16_t orc_mul_f2h_once(float a, float b) { return d2h((double)a * (double)b); }

ORC_API void orc_add_rms16_q35(float * x, const float * d, const float * nw, float eps, float * h, uint16_t * h16, int N, int n) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        float * xr = x + (size_t)t * N;
        if (d) for (int i = 0; i < N; i++) xr[i] = xr[i] + d[(size_t)t * N + i];
        const float scale = rsqrt_c(row_ss(xr, N) / (float)N + eps);
        for (int i = 0; i < N; i++) {
            const float tt = xr[i] * scale;
            h[(size_t)t * N + i] = tt * nw[i];
            h16[(size_t)t * N + i] = d2h((double)tt * (double)nw[i]);       /* one rounding from the last product, as the reference's binary */
        }
    }
}
/* the dense line's bf16-addend form: x = x + bf(d) (core.hip:57-61 promotion), then q35p_add_rms16's norm
 * (kernels/q35_prefill.hip:636-660), bf16 copy by to_bf16 (prefill_glue.hip:120-123). hbf / h optional. */
ORC_API void orc_add_rms_bf16(float * x, const uint16_t * d, const float * nw, float eps, float * h, uint16_t * hbf, int N, int n) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        float * xr = x + (size_t)t * N;
        if (d) for (int i = 0; i < N; i++) xr[i] = xr[i] + orc_bf2f(d[(size_t)t * N + i]);
        const float scale = rsqrt_c(row_ss(xr, N) / (float)N + eps);
        for (int i = 0; i < N; i++) {
            const float v = (xr[i] * scale) * nw[i];
            if (h) h[(size_t)t * N + i] = v;
            if (hbf) hbf[(size_t)t * N + i] = orc_to_bf16(v);
        }
    }
}
/* pf_rms_mul / OP_RMS_MUL (kernels/prefill_glue.hip:94-124, kernels/k3_gguf_ops.h:1233-1268): row r uses w[r % wr];
 * outputs optional: y fp32 (may alias x), ybf bf16, scl the row scale, q8 the q8_1 copy of y. */
ORC_API void orc_rms_mul(const float * x, const float * w, float * y, uint16_t * ybf, float * scl, uint8_t * q8,
                         int R, int wr, int K, float eps) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < R; r++) {
        const float * xr = x + (size_t)r * K, * wv = w + (size_t)(r % wr) * K;
        const float scale = rsqrt_c(row_ss(xr, K) / (float)K + eps);
        if (scl) scl[r] = scale;
        float hv[32];
        for (int i = 0; i < K; i++) {
            const float v = (xr[i] * scale) * wv[i];
            if (y) y[(size_t)r * K + i] = v;
            if (ybf) ybf[(size_t)r * K + i] = orc_to_bf16(v);
            if (q8) { hv[i & 31] = v; if ((i & 31) == 31) q8_1_block(hv, q8 + ((size_t)r * K + i) / 32 * 36); }
        }
    }
}
/* pf_hc_post_rms (kernels/prefill_glue.hip:130-170): per (token, stream) row q = t * HC + h of N values:
 * p = (1 / (1 + expf(-(inj[q] * rs)))) * 2 (contract off), res[q][i] = fmaf(b[t][i], p, res[q][i]) in place, then the
 * norm of the updated row with w[h]: xn fp32, xnbf bf16, scl the row scale, each optional. FP class through expf. */
ORC_API void orc_hc_post_rms(const float * b, const float * inj, float * res, const float * w, float * xn, uint16_t * xnbf,
                             float * scl, int T, int HC, int N, float rs, float eps) {
#pragma omp parallel for schedule(static)
    for (int q = 0; q < T * HC; q++) {
        const int h = q % HC, t = q / HC;
        float * rr = res + (size_t)q * N;
        const float * br = b + (size_t)t * N, * wv = w + (size_t)h * N;
        const float v = inj[q] * rs;
        const float sgm = 1.0f / (1.0f + expf(-v));
        const float p = sgm * 2.0f;
        for (int i = 0; i < N; i++) rr[i] = fmaf(br[i], p, rr[i]);
        const float scale = rsqrt_c(row_ss(rr, N) / (float)N + eps);
        if (scl) scl[q] = scale;
        for (int i = 0; i < N; i++) {
            const float y = (rr[i] * scale) * wv[i];
            if (xn) xn[(size_t)q * N + i] = y;
            if (xnbf) xnbf[(size_t)q * N + i] = orc_to_bf16(y);
        }
    }
}
/* pf_hc_post (kernels/prefill_glue.hip:172-188): the residual update alone, any D */
ORC_API void orc_hc_post(const float * b, const float * inj, float * res, int T, int HC, int D, float rs) {
#pragma omp parallel for schedule(static)
    for (int q = 0; q < T * HC; q++) {
        const int t = q / HC;
        const float v = inj[q] * rs;
        const float sgm = 1.0f / (1.0f + expf(-v));
        const float p = sgm * 2.0f;
        for (int i = 0; i < D; i++) res[(size_t)q * D + i] = fmaf(b[(size_t)t * D + i], p, res[(size_t)q * D + i]);
    }
}
/* pf_hc_mean (kernels/prefill_glue.hip:190-206): out[t][i] = rs * sum over h (fmaf chain from 0) of xn[t][h][i] *
 * (1 / (1 + expf(-g[t][h][i]))); xn given, or recomputed (scl, w given) as (x * scl[t * HC + h]) * w[h][i] */
ORC_API void orc_hc_mean(const float * x, const float * scl, const float * w, const float * g, float * out, int T, int HC, int D, float rs) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < T; t++)
        for (int i = 0; i < D; i++) {
            float sum = 0.0f;
            for (int h = 0; h < HC; h++) {
                const size_t o = ((size_t)t * HC + h) * D + i;
                const float xv = scl ? (x[o] * scl[t * HC + h]) * w[(size_t)h * D + i] : x[o];
                sum = fmaf(xv, 1.0f / (1.0f + expf(-g[o])), sum);
            }
            out[(size_t)t * D + i] = rs * sum;
        }
}
/* rmsnorm_f32 (kernels/core.hip:30-46): out = x * inv * w = (x * inv) * w; the squares accumulate by fmaf (the
 * reference's `s += x * x` under hipcc's default contraction) */
ORC_API void orc_rmsnorm_f32(const float * x, const float * w, float * out, int D, float eps, int rows) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++) {
        const float * xr = x + (size_t)r * D;
        const float inv = rsqrt_c(row_ss(xr, D) / (float)D + eps);
        for (int j = 0; j < D; j++) out[(size_t)r * D + j] = xr[j] * inv * w[j];
    }
}

/* ---- core.hip / fuse.hip elementwise --------------------------------------------------------------------------------- */
ORC_API void orc_embedding_f32(const int32_t * tok, const float * emb, float * out, int D, int T) {          /* core.hip:23-28 */
    for (int t = 0; t < T; t++) memcpy(out + (size_t)t * D, emb + (size_t)tok[t] * D, (size_t)D * 4);
}
ORC_API void orc_silu_mul_bf16(const uint16_t * gu, uint16_t * act, int H, int64_t n) {                      /* core.hip:48-55 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const int64_t r = i / H, c = i % H;
        const float g = orc_bf2f(gu[r * 2 * H + c]), u = orc_bf2f(gu[r * 2 * H + H + c]);
        const float s = rbf(g / (1.0f + expf(-g)));
        act[i] = orc_f2bf(s * u);
    }
}
ORC_API void orc_residual3(const float * x, const uint16_t * m, const uint16_t * y, float * out, int64_t n) { /* core.hip:57-61 */
    for (int64_t i = 0; i < n; i++) out[i] = (x[i] + orc_bf2f(m[i])) + orc_bf2f(y[i]);
}
ORC_API void orc_cast_bf16(const float * x, uint16_t * out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = orc_f2bf(x[i]); }
ORC_API void orc_copy_cols_bf16(const uint16_t * in, int ld_in, int c_in, uint16_t * out, int ld_out, int c_out, int n, int64_t rows) {
    for (int64_t r = 0; r < rows; r++) for (int c = 0; c < n; c++) out[r * ld_out + c_out + c] = in[r * ld_in + c_in + c];
}
/* residual_slices_bwd (kernels/fuse.hip:35-47) */
ORC_API void orc_residual_slices_bwd(const float * dout, const int32_t * pos, uint16_t * dm, uint16_t * dmlp, uint16_t * dys, int d, int64_t n) {
    for (int64_t e = 0; e < n; e++) {
        const uint16_t b = orc_f2bf(dout[e]);
        dm[e] = b; dmlp[e] = b;
        const int p = pos ? pos[e / d] : -1;
        if (p >= 0) dys[(size_t)p * d + e % d] = b;
    }
}
/* residual_slices_fwd (kernels/fuse.hip:19-33) */
ORC_API void orc_residual_slices_fwd(const float * x, const uint16_t * m, const uint16_t * mlp, const uint16_t * ys,
                                     const int32_t * pos, float * out, int d, int64_t n4) {
    for (int64_t e = 0; e < n4 * 4; e++) {
        const int r = (int)(e / d), c = (int)(e % d);
        const int p = pos ? pos[r] : -1;
        out[e] = ((x[e] + orc_bf2f(m[e])) + orc_bf2f(mlp[e])) + (p >= 0 ? orc_bf2f(ys[(size_t)p * d + c]) : 0.0f);
    }
}

/* ---- SwiGLU / gates ---------------------------------------------------------------------------------------------------- */
ORC_API void orc_swiglu16(const float * g, const float * u, uint16_t * y, int64_t n) {        /* k3_own_ops.h:258-262 */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) { const float gv = g[i]; y[i] = orc_f2h(gv / (1.0f + expf(-gv)) * u[i]); }
}
ORC_API void orc_silu_mul_f32(const float * g, const float * u, float * h, int64_t n) {       /* k3_gguf.hip:74-77 */
    for (int64_t i = 0; i < n; i++) h[i] = silu_f(g[i]) * u[i];
}
/* pf_gate_mul / q35p_gate_mul16 (prefill_attn.hip:379-386, q35_prefill.hip:960-969): y16 NULL -> fp32 out */
ORC_API void orc_gate_mul(const float * a, const float * gt, float * y, uint16_t * y16, int64_t N, int D, int stride, int off) {
    for (int64_t i = 0; i < N; i++) {
        const int64_t h = i / D; const int d = (int)(i - h * D);
        const float sgm = 1.0f / (1.0f + expf(-gt[(size_t)h * stride + off + d]));
        const float v = a[i] * sgm;
        if (y16) y16[i] = orc_f2h(v); else y[i] = v;
    }
}

/* ---- GDN short conv + L2 (prefill_glue.hip:314-341, prefill_gdn.hip:66-78) ---------------------------------------------- */
ORC_API void orc_gdn_conv(const float * x, const float * w, const float * st, float * y, int C, int T, int ldx, int ldy) {
    for (int t = 0; t < T; t++)
        for (int c = 0; c < C; c++) {
            float sumf = 0.0f;
            for (int j = 0; j < 4; j++) {
                const int tj = t - 3 + j;
                const float in = tj >= 0 ? x[(size_t)tj * ldx + c] : st[(size_t)c * 3 + 3 + tj];
                sumf = fmaf(in, w[(size_t)c * 4 + j], sumf);
            }
            y[(size_t)t * ldy + c] = silu_f(sumf);
        }
}
/* OP_GDN_CONV (kernels/k3_q35_ops.h:148-177): commit mprev tokens of xprev into the state, store it, convolve this pass's T tokens
 * from it without committing them, keep them as the next pass's xprev. (The sum of products is left to the compiler's contraction
 * in the reference: tolerance class; stated here as the fma chain of orc_gdn_conv.) */
ORC_API void orc_op_gdn_conv(const float * w, float * st, const float * x, const int32_t * params, float * y, float * xprev, int C, int T) {
    int mprev = params[1];
    mprev = mprev < 0 ? 0 : (mprev > T ? T : mprev);
    for (int c = 0; c < C; c++) {
        float s0 = st[(size_t)c * 3], s1 = st[(size_t)c * 3 + 1], s2 = st[(size_t)c * 3 + 2];
        for (int j = 0; j < mprev; j++) { s0 = s1; s1 = s2; s2 = xprev[(size_t)j * C + c]; }
        st[(size_t)c * 3] = s0; st[(size_t)c * 3 + 1] = s1; st[(size_t)c * 3 + 2] = s2;
        for (int t = 0; t < T; t++) {
            const float xv = x[(size_t)t * C + c];
            float sumf = 0.0f;
            sumf = fmaf(s0, w[(size_t)c * 4], sumf); sumf = fmaf(s1, w[(size_t)c * 4 + 1], sumf);
            sumf = fmaf(s2, w[(size_t)c * 4 + 2], sumf); sumf = fmaf(xv, w[(size_t)c * 4 + 3], sumf);
            y[(size_t)t * C + c] = silu_f(sumf);
            s0 = s1; s1 = s2; s2 = xv;
            xprev[(size_t)t * C + c] = xv;
        }
    }
}
ORC_API void orc_conv_state(const float * x, float * st, int C, int T, int ldx) {
    for (int c = 0; c < C; c++) {
        float s[3];
        for (int j = 0; j < 3; j++) { const int tj = T - 3 + j; s[j] = tj >= 0 ? x[(size_t)tj * ldx + c] : st[(size_t)c * 3 + 3 + tj]; }
        for (int j = 0; j < 3; j++) st[(size_t)c * 3 + j] = s[j];
    }
}
ORC_API void orc_gdn_l2(const float * x, float * y, int T, int heads, int K, int ldx, float rs) {
    for (int t = 0; t < T * heads; t++) {
        const int tt = t / heads, hh = t - tt * heads;
        const float * xr = x + (size_t)tt * ldx + (size_t)hh * K;
        const float scale = rsqrt_c(row_ss(xr, K) / (float)K + rs), s2 = 1.0f / sqrtf((float)K);
        for (int i = 0; i < K; i++) y[(size_t)t * K + i] = (scale * xr[i]) * s2;
    }
}

/* ---- QK-norm + rotary --------------------------------------------------------------------------------------------------- */
/* pf_qk_nr / OP_QK_NR (kernels/prefill_attn.hip:106-129, kernels/k3_gguf_ops.h:1495-1518): block t = row * heads + head.
 * The rotation is x0 c - x1 s / x0 s + x1 c as separately rounded products (the reference leaves contraction to the
 * compiler there: tolerance class). */
ORC_API void orc_qk_nr(const float * xin, int head_stride, int heads, const float * w, int D, int nrot,
                       float theta_scale, float eps, int pos0, float * out, int T) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < T * heads; t++) {
        const float * x = xin + (size_t)t * head_stride;
        float * y = out + (size_t)t * D;
        float nrm[512];
        const float scale = rsqrt_c(row_ss(x, D) / (float)D + eps);
        for (int i = 0; i < D; i++) nrm[i] = (scale * x[i]) * w[i];
        const float pos = (float)(pos0 + t / heads);
        for (int i = 0; i < D; i++) {
            if (i >= nrot) { y[i] = nrm[i]; continue; }
            const int j = i < nrot / 2 ? i : i - nrot / 2;
            const float theta = pos * powf(theta_scale, (float)j);
            const float c = cosf(theta), sn = sinf(theta);
            const float x0 = nrm[j], x1 = nrm[j + nrot / 2];
            y[i] = i < nrot / 2 ? x0 * c - x1 * sn : x0 * sn + x1 * c;
        }
    }
}

/* hadamard128 (python/caminus/ref_kv.py:72-89; kernels/own_kv_rot128.h:21-33) */
#define ROT128_SCALE 0x1.6a09e6p-4f
static void hadamard128(float * y) {
    for (int h = 1; h < 128; h <<= 1)
        for (int i = 0; i < 128; i++)
            if (!(i & h)) { const float a = y[i], b = y[i + h]; y[i] = a + b; y[i + h] = a - b; }
    for (int i = 0; i < 128; i++) y[i] = y[i] * ROT128_SCALE;
}
ORC_API void orc_hadamard128(const float * x, float * y, int64_t heads) {
    for (int64_t r = 0; r < heads; r++) { memcpy(y + r * 128, x + r * 128, 512); hadamard128(y + r * 128); }
}
/* pf_hadamard / OP_HADAMARD (kernels/prefill_attn.hip:132-153): in place, n in {64, 128, 256}, scale 1.0f / sqrtf(n) */
ORC_API void orc_hadamard_n(float * x, int64_t C, int n) {
    const float scale = 1.0f / sqrtf((float)n);
    for (int64_t c = 0; c < C; c++) {
        float * v = x + c * n;
        for (int h = 1; h < n; h <<= 1)
            for (int i = 0; i < n; i++)
                if (!(i & h)) { const float a = v[i], b = v[i + h]; v[i] = a + b; v[i + h] = a - b; }
        for (int i = 0; i < n; i++) v[i] = v[i] * scale;
    }
}

/* Q8 KV wire block (kernels/own_kv_codec.h:33-52; python/caminus/ref_kv.py:92-125): returns 1 when written, 0 refused */
static int kv_q8_encode(const float * x, uint8_t * y) {
    float amax = 0.0f; int finite = 1;
    for (int j = 0; j < 32; j++) { finite &= isfinite(x[j]) ? 1 : 0; amax = fmaxf(amax, fabsf(x[j])); }
    if (!finite) return 0;
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const uint16_t stored = orc_f2h(d);
    if (amax != 0.0f && (d == 0.0f || !isfinite(d) || !isfinite(inv) || (stored & 0x7c00u) == 0x7c00u)) return 0;
    memcpy(y, &stored, 2);
    for (int j = 0; j < 32; j++) y[2 + j] = (uint8_t)roundf_i8(x[j] * inv);
    return 1;
}
ORC_API void orc_kv_q8_encode(const float * x, uint8_t * y, uint8_t * ok, int64_t n) {
    for (int64_t i = 0; i < n; i++) ok[i] = (uint8_t)kv_q8_encode(x + i * 32, y + i * 34);
}
/* own_kv_q8_append (kernels/kv_codec.hip:10-30): err bits 1 span / 2 numeric / 4 layout */
ORC_API void orc_kv_q8_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0,
                              int rows, int T, int32_t * err) {
    if (M < 32 || M % 32 || ldk < M || ldv < M || rows < 1) { *err |= 4; return; }
    const int nb = M / 32;
    const size_t rb = (size_t)2 * nb * 34;
    for (int t = 0; t < T; t++) {
        const int64_t pos = (int64_t)pos0 + t;
        if (pos < 0 || pos >= rows) { *err |= 1; continue; }
        uint8_t * dst = cache + (size_t)pos * rb;
        for (int b = 0; b < 2 * nb; b++) {
            const float * x = (b < nb ? k + (size_t)t * ldk : v + (size_t)t * ldv) + (size_t)(b % nb) * 32;
            if (!kv_q8_encode(x, dst + (size_t)b * 34)) *err |= 2;
        }
    }
}
/* The Q8 KV reader: the decode of a wire block as the attention kernels do it (q3p_q8_stage, kernels/q3m_prefill.hip:617-632;
 * host reference decode_q8_kv, python/caminus/ref_kv.py:127-144): value = (float)code * (float)half scale, one fp32
 * multiply; f16: that value rounded to fp16 (the prefill staging). Row t = row_ids ? row_ids[t] : pos0 + t; a row outside
 * [0, rows) sets err bit 1 and leaves its outputs untouched. k, v: [T][ld] fp32 or fp16 bits. */
ORC_API void orc_kv_q8_read(const uint8_t * cache, const int32_t * row_ids, int pos0, int rows, int M, void * k, int ldk, void * v,
                            int ldv, int T, int f16, int32_t * err) {
    if (M < 32 || M % 32 || ldk < M || ldv < M || rows < 1) { *err |= 4; return; }
    const int nb = M / 32;
    const size_t rb = (size_t)2 * nb * 34;
    for (int t = 0; t < T; t++) {
        const int64_t pos = row_ids ? (int64_t)row_ids[t] : (int64_t)pos0 + t;
        if (pos < 0 || pos >= rows) { *err |= 1; continue; }
        const uint8_t * src = cache + (size_t)pos * rb;
        for (int b = 0; b < 2 * nb; b++) {
            const uint8_t * blk = src + (size_t)b * 34;
            uint16_t hd; memcpy(&hd, blk, 2);
            const float d = orc_h2f(hd);
            const size_t o = (b < nb ? (size_t)t * ldk : (size_t)t * ldv) + (size_t)(b % nb) * 32;
            for (int j = 0; j < 32; j++) {
                const float val = (float)(int8_t)blk[2 + j] * d;
                if (f16) ((uint16_t *)(b < nb ? k : v))[o + j] = orc_f2h(val); else ((float *)(b < nb ? k : v))[o + j] = val;
            }
        }
    }
}
/* pf_kv_append, q8_0 rows (kernels/prefill_attn.hip:157-181): no refusal rules; d stored as half, code by x * (1 / d) */
ORC_API void orc_pf_kv_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0,
                              int rows, int T, int32_t * err) {
    const int nb = M / 32;
    const size_t rb = (size_t)2 * nb * 34;
    for (int t = 0; t < T; t++) {
        const int pos = pos0 + t;
        if (pos < 0 || pos >= rows) { *err |= 1; continue; }
        for (int b = 0; b < 2 * nb; b++) {
            const float * x = (b < nb ? k + (size_t)t * ldk : v + (size_t)t * ldv) + (size_t)(b % nb) * 32;
            uint8_t * y = cache + (size_t)pos * rb + (size_t)b * 34;
            float amax = 0.0f;
            for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
            const float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
            const uint16_t hd = orc_f2h(d);
            memcpy(y, &hd, 2);
            for (int j = 0; j < 32; j++) y[2 + j] = (uint8_t)roundf_i8(x[j] * id);
        }
    }
}

/* q3p_qk_rope and q3p_qk_rope_q8 (kernels/q3m_prefill.hip:534-591), one call = n tokens.
 *   qkv fp32 [n][ldq] = q (nh heads) | k (nkv) | v (nkv), head dim 128. par = q_norm[128] | k_norm[128] | theta_scale |
 *   eps | (yarn: freq[64] | mscale). Token t sits at position pos ? pos[t] : pos0 + t.
 *   q8 = 0: q16 = fp16(rope(norm q)); cache row (fp16) = [K | V].
 *   q8 = 1: q16 = fp16(H f16r(rope)); cache row (bytes) = Q8 blocks of H f16r(rope(norm k)) | f16r(v).
 *   Row address: row_index(t) * row_bytes with row_index = position, or, paged (page_table != NULL):
 *   page_table[t * pt_stride + pos / page] * page + pos % page; a page id outside [0, n_pages) ORs 8 into err, a position outside
 *   the table row (or, unpaged with n_pages given as the cache's row count, outside the cache) ORs 1, and the row is not written
 *   (paging has no reference counterpart: each row's bytes equal the unpaged row's). */
ORC_API void orc_qk_rope(const float * qkv, int ldq, int nh, int nkv, const float * par, int pos0, const int32_t * pos,
                         uint16_t * q16, void * cache, int n, int yarn, int q8, int32_t * err,
                         const int32_t * page_table, int pt_stride, int page, int n_pages) {
    const size_t M = (size_t)nkv * 128;
    const size_t rb = q8 ? 2 * (M / 32) * 34 : 4 * M;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        const int p = pos ? pos[t] : pos0 + t;
        const float * row = qkv + (size_t)t * ldq;
        const float eps = par[257];
        float rc[64], rs[64];
        for (int i = 0; i < 64; i++) {
            if (yarn) { const float theta = (float)p * par[258 + i], ms = par[322]; rc[i] = cosf(theta) * ms; rs[i] = sinf(theta) * ms; }
            else { const float theta = (float)p * powf(par[256], (float)i); rc[i] = cosf(theta); rs[i] = sinf(theta); }
        }
        uint8_t * cw = NULL;
        /* our addressing layer's span refusal: a position outside the sequence's table row, or (unpaged, n_pages = rows of the cache when
         * given) outside the cache: bit 1, the row is not written */
        const int span = p >= 0 && (page_table ? p / page < pt_stride : (n_pages == 0 || p < n_pages));
        if (!span) {
#pragma omp atomic
            *err |= 1;
        } else if (page_table) {
            const int pg = page_table[(size_t)t * pt_stride + p / page];
            if (pg < 0 || pg >= n_pages) {
#pragma omp atomic
                *err |= 8;
            } else cw = (uint8_t *)cache + ((size_t)pg * page + (size_t)(p % page)) * rb;
        } else cw = (uint8_t *)cache + (size_t)p * rb;
        for (int hy = 0; hy < nh + nkv; hy++) {
            const int isq = hy < nh, g = hy - nh;
            const float * x = isq ? row + (size_t)hy * 128 : row + (size_t)nh * 128 + (size_t)g * 128;
            const float * wn = isq ? par : par + 128;
            float y1[128], y[128];
            const float scale = rsqrt_c(row_ss(x, 128) / 128 + eps);
            for (int i = 0; i < 128; i++) y1[i] = (scale * x[i]) * wn[i];
            for (int i = 0; i < 64; i++) {
                y[i] = fmaf(y1[i], rc[i], -(y1[i + 64] * rs[i]));
                y[i + 64] = fmaf(y1[i + 64], rc[i], y1[i] * rs[i]);
            }
            if (q8) { for (int i = 0; i < 128; i++) y[i] = f16r(y[i]); hadamard128(y); }
            if (isq) { for (int i = 0; i < 128; i++) q16[((size_t)t * nh + hy) * 128 + i] = orc_f2h(y[i]); continue; }
            if (!cw) continue;
            const float * vv = row + (size_t)nh * 128 + M + (size_t)g * 128;
            if (!q8) {
                uint16_t * c16 = (uint16_t *)cw;
                for (int i = 0; i < 128; i++) { c16[(size_t)g * 128 + i] = orc_f2h(y[i]); c16[M + (size_t)g * 128 + i] = orc_f2h(vv[i]); }
            } else {
                float v16[128];
                for (int i = 0; i < 128; i++) v16[i] = f16r(vv[i]);
                for (int b = 0; b < 4; b++) {
                    int bad = !kv_q8_encode(y + 32 * b, cw + ((size_t)g * 4 + b) * 34);
                    bad |= !kv_q8_encode(v16 + 32 * b, cw + (M / 32 + (size_t)g * 4 + b) * 34);
                    if (bad) {
#pragma omp atomic
                        *err |= 2;
                    }
                }
            }
        }
    }
}

/* ---- quantized embedding rows (kernels/q3m_prefill.hip:364-380; python/caminus/own_dequant.py:28-37,202-206) ---------- */
ORC_API void orc_emb_q4k(const uint8_t * W, int rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        int tok = toks[t]; tok = tok < 0 ? 0 : tok; tok = tok > vocab - 1 ? vocab - 1 : tok;
        const uint8_t * row = W + (size_t)tok * rb;
        for (int i = 0; i < N; i++) {
            const uint8_t * blk = row + (size_t)(i >> 8) * 144;
            const int j = i & 255, sb = j >> 5, l = j & 31, is = sb >> 1, hi = sb & 1;
            const uint8_t * s = blk + 4;
            const uint32_t sc = sb < 4 ? (s[sb] & 63u) : ((s[sb + 4] & 0xfu) | ((uint32_t)(s[sb - 4] >> 6) << 4));
            const uint32_t m = sb < 4 ? (s[sb + 4] & 63u) : ((uint32_t)(s[sb + 4] >> 4) | ((uint32_t)(s[sb] >> 6) << 4));
            const float d = orc_h2f((uint16_t)(blk[0] | (blk[1] << 8))), dm = orc_h2f((uint16_t)(blk[2] | (blk[3] << 8)));
            const float q = (float)((blk[16 + is * 32 + l] >> (4 * hi)) & 15);
            const float a = d * (float)sc, b = a * q, c = dm * (float)m;
            const float v = b - c;
            if (x) x[(size_t)t * N + i] = v;
            if (xbf) xbf[(size_t)t * N + i] = orc_f2bf(v);
        }
    }
}
ORC_API void orc_emb_q8_0(const uint8_t * W, int rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n) {
#pragma omp parallel for schedule(static)
    for (int t = 0; t < n; t++) {
        int tok = toks[t]; tok = tok < 0 ? 0 : tok; tok = tok > vocab - 1 ? vocab - 1 : tok;
        const uint8_t * row = W + (size_t)tok * rb;
        for (int i = 0; i < N; i++) {
            const uint8_t * blk = row + (size_t)(i >> 5) * 34;
            const float d = orc_h2f((uint16_t)(blk[0] | (blk[1] << 8)));
            const float v = d * (float)(int8_t)blk[2 + (i & 31)];
            if (x) x[(size_t)t * N + i] = v;
            if (xbf) xbf[(size_t)t * N + i] = orc_f2bf(v);
        }
    }
}

/* IQ4_XS rows (kernels/prefill_feed.hip:40-54): one value at a time; err bit 1 for an id outside the table (clamped) */
static const float KV_IQ4[16] = {-127.f, -104.f, -83.f, -65.f, -49.f, -35.f, -22.f, -10.f, 1.f, 13.f, 25.f, 38.f, 53.f, 69.f, 89.f, 113.f};
ORC_API void orc_emb_iq4xs(const uint8_t * W, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int nblk, int n, int * err) {
    const int D = nblk * 256;
    for (int p = 0; p < n; p++) {
        int t = toks[p];
        if (t < 0 || t >= vocab) { if (err) *err |= 2; t = t < 0 ? 0 : vocab - 1; }
        for (int k = 0; k < D; k++) {
            const int bl = k >> 8, w = k & 255, ib = w >> 5, j = w & 31;
            const uint8_t * b = W + (size_t)t * (size_t)(nblk * 136) + (size_t)bl * 136;
            const int sh = b[2] | (b[3] << 8), sl = b[4 + (ib >> 1)];
            const int ls = ((sl >> ((ib & 1) * 4)) & 15) | (((sh >> (2 * ib)) & 3) << 4);
            const float dl = orc_h2f((uint16_t)(b[0] | (b[1] << 8))) * (float)(ls - 32);
            const uint8_t q = b[8 + 16 * ib + (j & 15)];
            const float v = dl * KV_IQ4[j < 16 ? (q & 15) : (q >> 4)];
            if (x) x[(size_t)p * D + k] = v;
            if (xbf) xbf[(size_t)p * D + k] = orc_f2bf(v);
        }
    }
}
/* IQ4_NL feed rows (kernels/prefill_feed.hip:24-35); err bit 0 for an index outside [0, nuniq) (clamped) */
ORC_API void orc_ple_rows_iq4nl(const uint8_t * raw, const int32_t * inv, int nuniq, int nrows, int bpr, float * out, int * err) {
    const int hd = bpr * 32;
    for (int r = 0; r < nrows; r++) {
        int u = inv[r];
        if (u < 0 || u >= nuniq) { *err |= 1; u = u < 0 ? 0 : nuniq - 1; }
        for (int k = 0; k < hd; k++) {
            const int b = k >> 5, j = k & 31;
            const uint8_t * blk = raw + (size_t)u * (size_t)(bpr * 18) + (size_t)b * 18;
            const uint8_t q = blk[2 + (j & 15)];
            out[(size_t)r * hd + k] = orc_h2f((uint16_t)(blk[0] | (blk[1] << 8))) * KV_IQ4[j < 16 ? (q & 15) : (q >> 4)];
        }
    }
}
/* IQ2_S rows (kernels/k3_q35t_ops.h:163-174); grid: [1024][8] magnitude bytes (the caller's copy of the format's codebook) */
ORC_API void orc_emb_iq2s(const uint8_t * W, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n, const uint8_t * grid) {
    for (int p = 0; p < n; p++) {
        int t = toks[p]; t = t < 0 ? 0 : t; t = t > vocab - 1 ? vocab - 1 : t;
        const uint8_t * row = W + (size_t)t * (size_t)(N / 256 * 82);
        for (int i = 0; i < N; i++) {
            const uint8_t * blk = row + (size_t)(i >> 8) * 82;
            const int j = i & 255, ib = j >> 5, g = (j >> 3) & 3, k = j & 7;
            const float d = orc_h2f((uint16_t)(blk[0] | (blk[1] << 8)));
            const uint32_t idx = blk[2 + 4 * ib + g] | (((uint32_t)(blk[66 + ib] >> (2 * g)) & 3u) << 8);
            const float mag = (float)grid[idx * 8 + k];
            const float sc = (float)((blk[74 + ib] >> (4 * ((j >> 4) & 1))) & 15);
            const float db = (d * (0.5f + sc)) * 0.25f;
            const float v0 = db * mag, v = ((blk[34 + (j >> 3)] >> k) & 1) ? -v0 : v0;
            if (x) x[(size_t)p * N + i] = v;
            if (xbf) xbf[(size_t)p * N + i] = orc_f2bf(v);
        }
    }
}

/* ---- activation fake-quant (kernels/actq.hip:40-53, 96-132, 247-274, 307-310). Pinned against a torch graph (see header). - */
#define HSCALE 0.08837890625f
static void fwht128_actq(float * v) {   /* chunk element e = 4 lane + r: stages inside a lane's 4, then lanes by m = 1..16 */
    for (int l = 0; l < 32; l++) {
        float * p = v + 4 * l; float a, b;
        a = p[0]; b = p[1]; p[0] = a + b; p[1] = a - b;
        a = p[2]; b = p[3]; p[2] = a + b; p[3] = a - b;
        a = p[0]; b = p[2]; p[0] = a + b; p[2] = a - b;
        a = p[1]; b = p[3]; p[1] = a + b; p[3] = a - b;
    }
    float n[128];
    for (int m = 1; m < 32; m <<= 1) {
        for (int l = 0; l < 32; l++)
            for (int e = 0; e < 4; e++) { const float own = v[4 * l + e], p = v[4 * (l ^ m) + e]; n[4 * l + e] = (l & m) ? (p - own) : (own + p); }
        memcpy(v, n, sizeof n);
    }
}
/* src 0: fp32 x [M][K]; 1: bf16 x; 2: silu-mul of gu (bf16, row stride ld, F = K); 3: RMSNorm source (x fp32, nw, rstd) */
static void actq_row(const float * u_in, int K, float clip, int qmax, uint16_t * y, float * s_out, uint8_t * codes) {
    float u[8192];
    float amax = 0.0f;
    for (int ch = 0; ch < K / 128; ch++) {
        float * c = u + ch * 128;
        for (int e = 0; e < 128; e++) c[e] = rbf(u_in[ch * 128 + e]);
        fwht128_actq(c);
        for (int e = 0; e < 128; e++) { c[e] = rbf(c[e] * HSCALE); amax = fmaxf(amax, fabsf(c[e])); }
    }
    const float s = fmaxf(amax * clip / (float)qmax, 1e-8f);
    if (s_out) *s_out = s;
    for (int k = 0; k < K; k++) {
        const float q = fminf(fmaxf(rintf(u[k] / s), (float)(-qmax - 1)), (float)qmax);
        if (y) y[k] = orc_f2bf(q * s);
        if (codes) {
            const uint8_t nib = (uint8_t)((uint32_t)(int)q & 0xfu);
            if (k & 1) codes[k / 2] = (uint8_t)(codes[k / 2] | (nib << 4)); else codes[k / 2] = nib;
        }
    }
}
ORC_API void orc_actq_fwd(const void * x, int is_bf16, uint16_t * y, float * s, uint8_t * codes, int M, int K, float clip, int qmax) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        float src[8192];
        for (int k = 0; k < K; k++) src[k] = is_bf16 ? orc_bf2f(((const uint16_t *)x)[(size_t)r * K + k]) : ((const float *)x)[(size_t)r * K + k];
        actq_row(src, K, clip, qmax, y ? y + (size_t)r * K : NULL, s ? s + r : NULL, codes ? codes + (size_t)r * (K / 2) : NULL);
    }
}
ORC_API void orc_silu_mul_actq_fwd(const uint16_t * gu, int ld, int F, uint16_t * y, float * s, uint8_t * codes, int M, float clip, int qmax) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        float src[8192];
        const uint16_t * row = gu + (size_t)r * ld;
        for (int k = 0; k < F; k++) { const float g = orc_bf2f(row[k]); src[k] = rbf(rbf(g / (1.0f + expf(-g))) * orc_bf2f(row[F + k])); }
        actq_row(src, F, clip, qmax, y ? y + (size_t)r * F : NULL, s ? s + r : NULL, codes ? codes + (size_t)r * (F / 2) : NULL);
    }
}
/* block_entry_fwd (actq.hip:247-274): rstd from the contract tree; source x * rstd * nw; nab gate projections
 * ab[j] = bf16(sum_k bf16(h_k) wab[j][k]) with the 256-thread tree (thread-strided fmaf-free `acc += hb * w` is left to
 * the compiler's contraction in the reference; the contract here is fmaf) */
ORC_API void orc_block_entry_fwd(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y,
                                 float * s, uint8_t * codes, uint16_t * ab, float * rstd_out, int M, int d, float clip, int qmax) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        const float * xr = x + (size_t)r * d;
        const float rstd = rsqrt_c(row_ss(xr, d) / (float)d + eps);
        if (rstd_out) rstd_out[r] = rstd;
        float src[8192];
        for (int k = 0; k < d; k++) src[k] = xr[k] * rstd * nw[k];
        actq_row(src, d, clip, qmax, y ? y + (size_t)r * d : NULL, s ? s + r : NULL, codes ? codes + (size_t)r * (d / 2) : NULL);
        for (int j = 0; j < nab; j++) {
            float part[256];
            for (int t = 0; t < 256; t++) part[t] = 0.0f;
            for (int k = 0; k < d; k++) part[k & 255] = fmaf(rbf(src[k]), orc_bf2f(wab[(size_t)j * d + k]), part[k & 255]);
            float tot = 0.0f;
            for (int g = 0; g < 8; g++) tot += bfly32_sum(part + 32 * g);
            ab[(size_t)r * nab + j] = orc_f2bf(tot);
        }
    }
}

/* ---- activation fake-quant, backward (kernels/actq.hip:134-218, 275-313). Pinned against autograd (see header). ---------
 * Sum tree: logical thread (w = chunk % 8, l = element / 4 % 32) adds its terms in chunk order with fmaf; the 32 threads
 * of a w combine by xor 16 .. 1; the eight w sums are added in order. out: the bf16-valued gradient of the bf16 source. */
static float tree8x32(const float * part /* [8][32] */) {
    float r = bfly32_sum(part);
    for (int w = 1; w < 8; w++) r += bfly32_sum(part + 32 * w);
    return r;
}
static void actq_bwd_row(const float * src, const uint16_t * g, int K, float clip, int qmax, float * out) {
    float u[8192];
    float amax = 0.0f;
    for (int ch = 0; ch < K / 128; ch++) {
        float * c = u + ch * 128;
        for (int e = 0; e < 128; e++) c[e] = rbf(src[ch * 128 + e]);
        fwht128_actq(c);
        for (int e = 0; e < 128; e++) { c[e] = rbf(c[e] * HSCALE); amax = fmaxf(amax, fabsf(c[e])); }
    }
    const float s_raw = amax * clip / (float)qmax, s = fmaxf(s_raw, 1e-8f);
    const float lo = (float)(-qmax - 1), hi = (float)qmax;
    float dl[256], ti[256];
    for (int t = 0; t < 256; t++) dl[t] = ti[t] = 0.0f;
    for (int ch = 0; ch < K / 128; ch++)
        for (int e = 0; e < 128; e++) {
            const int k = ch * 128 + e, th = 32 * (ch % 8) + e / 4;
            const float t = u[k] / s, r = rintf(t), q = fminf(fmaxf(r, lo), hi);
            const int m = r > lo && r < hi;
            dl[th] = fmaf(orc_bf2f(g[k]), m ? q - t : q, dl[th]);
            ti[th] += fabsf(u[k]) == amax ? 1.0f : 0.0f;
        }
    const float dlds = tree8x32(dl), ties = tree8x32(ti);
    const float coef = s_raw >= 1e-8f ? dlds * clip / (float)qmax / ties : 0.0f;
    for (int ch = 0; ch < K / 128; ch++) {
        float d[128];
        for (int e = 0; e < 128; e++) {
            const int k = ch * 128 + e;
            const float t = u[k] / s, r = rintf(t);
            float v = orc_bf2f(g[k]) * (r > lo && r < hi ? 1.0f : 0.0f);
            if (fabsf(u[k]) == amax && u[k] != 0.0f) v += u[k] > 0.0f ? coef : -coef;
            d[e] = rbf(v);
        }
        fwht128_actq(d);
        for (int e = 0; e < 128; e++) out[ch * 128 + e] = rbf(d[e] * HSCALE);
    }
}
ORC_API void orc_actq_rotate(const uint16_t * x, uint16_t * u, int M, int K) {
    for (int r = 0; r < M; r++)
        for (int ch = 0; ch < K / 128; ch++) {
            float c[128];
            for (int e = 0; e < 128; e++) c[e] = orc_bf2f(x[(size_t)r * K + ch * 128 + e]);
            fwht128_actq(c);
            for (int e = 0; e < 128; e++) u[(size_t)r * K + ch * 128 + e] = orc_f2bf(c[e] * HSCALE);
        }
}
ORC_API void orc_actq_bwd(const void * x, int is_bf16, const uint16_t * g, void * dx, int M, int K, float clip, int qmax) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        float src[8192], out[8192];
        for (int k = 0; k < K; k++) src[k] = is_bf16 ? orc_bf2f(((const uint16_t *)x)[(size_t)r * K + k]) : ((const float *)x)[(size_t)r * K + k];
        actq_bwd_row(src, g + (size_t)r * K, K, clip, qmax, out);
        for (int k = 0; k < K; k++) { if (is_bf16) ((uint16_t *)dx)[(size_t)r * K + k] = orc_f2bf(out[k]); else ((float *)dx)[(size_t)r * K + k] = out[k]; }
    }
}
/* silu_mul_actq_bwd (actq.hip:140-153, 311-314): dgu [M][2F] = [dg | du]. tab = 0: the sigmoid of silu's derivative from the C library's
 * expf, as the reference's source reads. tab = 1: from ex = (float)exp(-(double)g), the correctly rounded single-precision exponential: the
 * definition of the 65536-entry table the HIP kernel reads (one entry per bf16 gate), restated here so that dg can be compared bit for bit.
 * The two differ where glibc's expf is not correctly rounded (rare; at most one bf16 step in dg). The reference holds no fixture for this
 * gradient: parity of dg with the reference's own device expf is unpinned beyond that step. */
static void silu_mul_actq_bwd_impl(const uint16_t * gu, int ld, int F, const uint16_t * g, uint16_t * dgu, int M, float clip, int qmax, int tab) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        float src[8192], out[8192];
        const uint16_t * row = gu + (size_t)r * ld;
        for (int k = 0; k < F; k++) { const float gg = orc_bf2f(row[k]); src[k] = rbf(rbf(gg / (1.0f + expf(-gg))) * orc_bf2f(row[F + k])); }
        actq_bwd_row(src, g + (size_t)r * F, F, clip, qmax, out);
        for (int k = 0; k < F; k++) {
            const float dact = out[k], gg = orc_bf2f(row[k]), uu = orc_bf2f(row[F + k]);
            const float ex = expf(-gg), sl = rbf(gg / (1.0f + ex)), ds = rbf(dact * uu);
            const float sig = 1.0f / (1.0f + (tab ? (float)exp(-(double)gg) : ex));
            dgu[(size_t)r * 2 * F + k] = orc_f2bf(ds * sig * fmaf(gg, 1.0f - sig, 1.0f));
            dgu[(size_t)r * 2 * F + F + k] = orc_f2bf(dact * sl);
        }
    }
}
ORC_API void orc_silu_mul_actq_bwd(const uint16_t * gu, int ld, int F, const uint16_t * g, uint16_t * dgu, int M, float clip, int qmax) {
    silu_mul_actq_bwd_impl(gu, ld, F, g, dgu, M, clip, qmax, 0);
}
ORC_API void orc_silu_mul_actq_bwd_tab(const uint16_t * gu, int ld, int F, const uint16_t * g, uint16_t * dgu, int M, float clip, int qmax) {
    silu_mul_actq_bwd_impl(gu, ld, F, g, dgu, M, clip, qmax, 1);
}
/* block_entry_bwd (actq.hip:275-304): thread t = k % 256 adds dot terms in k order with fmaf; 8 x 32 tree; d <= 1024 */
ORC_API void orc_block_entry_bwd(const float * x, const float * nw, const float * rstd_in, const uint16_t * wab, int nab, const uint16_t * dy,
                                 const uint16_t * dab, float * dx, int M, int d, float clip, int qmax) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < M; r++) {
        const float * xr = x + (size_t)r * d;
        const float rstd = rstd_in[r];
        float src[1024], dh[1024], part[256];
        for (int k = 0; k < d; k++) src[k] = xr[k] * rstd * nw[k];
        actq_bwd_row(src, dy + (size_t)r * d, d, clip, qmax, dh);
        for (int t = 0; t < 256; t++) part[t] = 0.0f;
        const int half = nab / 2;
        for (int k = 0; k < d; k++) {
            float gk = dh[k];
            if (nab) {
                float pa = 0.0f, pb = 0.0f;
                for (int j = 0; j < half; j++) pa = fmaf(orc_bf2f(dab[(size_t)r * nab + j]), orc_bf2f(wab[(size_t)j * d + k]), pa);
                for (int j = half; j < nab; j++) pb = fmaf(orc_bf2f(dab[(size_t)r * nab + j]), orc_bf2f(wab[(size_t)j * d + k]), pb);
                gk = (gk + rbf(pa)) + rbf(pb);
            }
            dh[k] = gk;
            part[k & 255] = fmaf(gk * nw[k], xr[k] * rstd, part[k & 255]);
        }
        const float dot = tree8x32(part) / (float)d;
        for (int k = 0; k < d; k++) dx[(size_t)r * d + k] = rstd * (dh[k] * nw[k] - (xr[k] * rstd) * dot);
    }
}

/* ---- more row kernels of the batched prefill -----------------------------------------------------------------------------
 * pf_gdn_norm / q35p_gdn_norm16 (prefill_gdn.hip:385-407, q35_prefill.hip:671-692): contraction off, so the row sum is a
 * product and a sum per element in thread t = i % 256's chain; the 8 x 32 tree; rsqrtf -> 1 / sqrt. */
ORC_API void orc_gdn_norm(const float * o, const float * w, const float * z, float * y, uint16_t * y16, int K, float eps, long rows, int silu) {
    for (long r = 0; r < rows; r++) {
        const float * orow = o + r * K, * zr = z + r * K;
        float part[256];
        for (int t = 0; t < 256; t++) part[t] = 0.0f;
        for (int i = 0; i < K; i++) { const float p = orow[i] * orow[i]; part[i & 255] = part[i & 255] + p; }
        float tot = 0.0f;
        for (int g = 0; g < 8; g++) tot += bfly32_sum(part + 32 * g);
        const float scale = rsqrt_c(tot / (float)K + eps);
        for (int i = 0; i < K; i++) {
            const float a = scale * orow[i], nrm = a * w[i];
            float gate;
            if (silu) { const float e = 1.0f + expf(-zr[i]); gate = zr[i] / e; } else { const float e = 1.0f + expf(-zr[i]); gate = 1.0f / e; }
            const float v = nrm * gate;
            if (y) y[r * K + i] = v;
            if (y16) y16[r * K + i] = orc_f2h(v);
        }
    }
}
ORC_API void orc_gdn_gates(const float * al, int lda, const float * be, int ldb, const float * dt, const float * A, float * y, int H, int T) {
    for (int tt = 0; tt < T; tt++)
        for (int h = 0; h < H; h++) {
            const float ab = al[(size_t)tt * lda + h] + dt[h];
            const float sp = ab > 20.0f ? ab : logf(1.0f + expf(ab));
            y[(size_t)tt * 2 * H + h] = sp * A[h];
            y[(size_t)tt * 2 * H + H + h] = 1.0f / (1.0f + expf(-be[(size_t)tt * ldb + h]));
        }
}
ORC_API void orc_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, int rows, int * err, int T) {
    for (int tt = 0; tt < T; tt++) {
        const long pos = (long)pos0 + tt;
        if (pos < 0 || pos >= rows) { *err |= 1; continue; }
        for (int i = 0; i < M; i++) { cache[(size_t)pos * 2 * M + i] = orc_f2h(k[(size_t)tt * ldk + i]); cache[(size_t)pos * 2 * M + M + i] = orc_f2h(v[(size_t)tt * ldv + i]); }
    }
}
/* OP_OWN_MOE_SUM (kernels/k3_own_ops.h:263-271) */
ORC_API void orc_own_moe_sum(const float * d, const float * w, float * x, long n, int S) {
    for (long i = 0; i < n; i++) {
        float acc = 0.0f;
        for (int s = 0; s < S; s++) acc = w ? fmaf(w[s], d[(size_t)s * n + i], acc) : acc + d[(size_t)s * n + i];
        x[i] += acc;
    }
}
/* OP_SHEXP_ADD (kernels/k3_gguf_ops.h:1220-1229) */
ORC_API void orc_shexp_add(const float * moe, const float * sh, const float * logit, float * out, long n, int T) {
    const long dd = n / T;
    for (long i = 0; i < n; i++) {
        const float s = 1.0f / (1.0f + expf(-logit[i / dd]));
        const float g = sh[i] * s;
        out[i] = moe[i] + g;
    }
}
ORC_API void orc_add_sum(const float * a, const float * b, float * y, long n) { for (long i = 0; i < n; i++) { const float ab = a[i] + b[i]; y[i] = y[i] + ab; } }
static inline uint16_t to_bf16_plain(float v) { const uint32_t u = f2u(v); return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }
ORC_API void orc_to_bf16_rows(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, float rs, int silu) {
    for (int t = 0; t < Tpad; t++)
        for (int j = 0; j < K; j++) {
            uint16_t o = 0;
            if (t < T) {
                float v = x[(size_t)t * ldx + j];
                if (silu) { const float s = fmaf(rs, v, 0.0f); v = s / (1.0f + expf(-s)); }
                o = to_bf16_plain(v);
            }
            y[(size_t)t * K + j] = o;
        }
}
ORC_API void orc_hc_avg(const float * r, float * y, int T, int hc, int D, int ldo) {
    for (int tt = 0; tt < T; tt++)
        for (int i = 0; i < D; i++) {
            float acc = r[(size_t)(tt * hc) * D + i];
            for (int h = 1; h < hc; h++) acc = acc + r[(size_t)(tt * hc + h) * D + i];
            y[(size_t)tt * ldo + i] = acc * (1.0f / (float)hc);
        }
}
/* pf_ple_gate (prefill_glue.hip:343-372) */
ORC_API void orc_ple_gate(const float * kn, const float * q, const float * qscl, const float * qw, const float * val, int ldv, float * gated,
                          float * gate_out, int HC, int D, int T) {
    for (int tt = 0; tt < T; tt++) {
        float gate[8];
        for (int st = 0; st < HC; st++) {
            float part[256];
            for (int t = 0; t < 256; t++) part[t] = 0.0f;
            for (int i = 0; i < D; i++) {
                const size_t o = ((size_t)tt * HC + st) * D + i;
                const float qv = qscl ? (q[o] * qscl[tt * HC + st]) * qw[(size_t)st * D + i] : q[o];
                const float p = kn[o] * qv;
                part[i & 255] = part[i & 255] + p;
            }
            float sum = 0.0f;
            for (int g = 0; g < 8; g++) sum += bfly32_sum(part + 32 * g);
            const float s = sum * (1.0f / sqrtf((float)D));
            const float mag = sqrtf(fmaxf(fabsf(s), 1e-6f));
            const float sgn = s > 0.0f ? 1.0f : (s < 0.0f ? -1.0f : 0.0f);
            gate[st] = 1.0f / (1.0f + expf(-(sgn * mag)));
            gate_out[tt * HC + st] = gate[st];
        }
        for (int c = 0; c < HC * D; c++) gated[(size_t)tt * HC * D + c] = val[(size_t)tt * ldv + c % D] * gate[c / D];
    }
}
/* pf_ple_conv / pf_ple_hist (prefill_glue.hip:374-414); w: fp16 bits [C][4] */
static float ple_x_c(const float * x, const float * xscl, const float * xw, int tb, int c, int C, int D) {
    return xscl ? (x[(size_t)tb * C + c] * xscl[tb * (C / D) + c / D]) * xw[c] : x[(size_t)tb * C + c];
}
ORC_API void orc_ple_conv(const float * x, const float * xscl, const float * xw, const uint16_t * w, const float * hist, float * y, const float * a,
                          float * res, int C, int T, int D, int dil) {
    const int hl = 3 * dil;
    for (int t = 0; t < T; t++)
        for (int c = 0; c < C; c++) {
            float conv = 0.0f;
            for (int k = 0; k < 4; k++) {
                const int back = (3 - k) * dil;
                const float xv = back <= t ? ple_x_c(x, xscl, xw, t - back, c, C, D) : hist[(size_t)c * hl + hl - (back - t)];
                const float term = xv * orc_h2f(w[(size_t)c * 4 + k]);
                conv = k == 0 ? term : conv + term;
            }
            const float o = conv / (1.0f + expf(-conv));
            const size_t i = (size_t)t * C + c;
            if (y) y[i] = o;
            if (res) { const float ab = a[i] + o; res[i] = res[i] + ab; }
        }
}
ORC_API void orc_ple_hist(const float * x, const float * xscl, const float * xw, float * hist, int C, int T, int D, int dil) {
    const int hl = 3 * dil;
    for (int c = 0; c < C; c++) {
        float h[32];
        for (int j = 0; j < hl; j++) { const int tj = T - hl + j; h[j] = tj < 0 ? hist[(size_t)c * hl + hl + tj] : ple_x_c(x, xscl, xw, tj, c, C, D); }
        for (int j = 0; j < hl; j++) hist[(size_t)c * hl + j] = h[j];
    }
}

ORC_API int orc_version(void) { return 1; }
