/* camx.h - C ABI of libcamx.so: the fused per-layer row kernels of the Caminus inference engine for AMD Instinct MI355X
 * (gfx950). Plain pointers and sizes, no C++ or PyTorch types. Every pointer is a device pointer unless said otherwise.
 *
 * Conventions
 *   - Every entry point queues work on `stream` (a hipStream_t; NULL = the default stream) and returns at once:
 *     0, or a hipError_t value (1 = invalid value: a shape, alignment or pointer argument was refused and nothing was
 *     launched). camx_error_string() names the value.
 *   - The library allocates nothing per call and keeps no state between calls, except a 128 KiB lookup table of
 *     bf16(silu(g)) for every bf16 g that camx_swiglu_mmq_q8_1, camx_silu_mul_bf16 and camx_silu_mul_actq_fwd / _bwd share and
 *     that camx_init(), or else the first of them to be called, fills once per device (that call waits for its stream once: call
 *     camx_init() before any graph capture). All four therefore produce the same activation bits for a row, whatever the batch size.
 *   - bf16 / fp16 values travel as uint16_t bit patterns. "rows" / "n" / "T" arguments that the reference kernels took
 *     from their launch grid are explicit trailing arguments here.
 *   - Device-side errors are sticky int32 words OR-ed by the kernels and never cleared by them; bit meanings are given at
 *     each function.
 *   - Each declaration cites the reference kernel or op it replaces (paths relative to the reference checkout).
 *
 * Numeric contract (see oracle/camx_oracle.c for the executable statement): sums of squares are formed as the reference
 * forms them (256 logical threads, fmaf chains in element order, 32-lane xor butterfly, 8 group sums in order); rsqrt is
 * 1 / sqrt with IEEE square root and division; quantizer outputs (q8_1, MMQ q8_1, Q8 KV blocks, actq codes), Hadamard
 * transforms and GGUF dequantization are bit-exact; values that pass through expf / cosf / sinf are within 1e-5 relative
 * (fp32 outputs) or one unit in the last place (fp16 / bf16 outputs).
 */
#ifndef CAMX_H
#define CAMX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t * camx_stream_t;      /* = hipStream_t */

/* ---- library ---------------------------------------------------------------------------------------------------------- */
int camx_version(void);
const char * camx_arch(void);                     /* "gfx950" */
const char * camx_error_string(int err);          /* hipGetErrorString; replaces device/hip.py:35-37's lookup */
/* Fills the current device's lookup tables (bf16(silu g), the fused backward's sigmoid, their LDS extracts) on `stream` and waits for it
 * once; afterwards no entry point synchronizes on this device, so every later call may sit inside a stream capture (the reference loads
 * its code objects before it captures: python/caminus/prefill/attn.py:150-155). Idempotent and thread-safe. Without it the first call of
 * an entry point that needs a table does the same work. */
int camx_init(camx_stream_t stream);

/* ---- residual add + RMSNorm -------------------------------------------------------------------------------------------- */
/* q3p_add_rms16 (kernels/q3m_prefill.hip:385-415) = OP_OWN_ADD_RMS16 (kernels/k3_own_ops.h:326-383).
 * Per token t < n: x[t] += sum over slots s < S of w[t][s] * d[t][s] (fma in slot order from 0; w NULL: acc + d; S = 0 or
 * d NULL: no add), x written back; h = (x * scale) * nw, h16 = fp16(h). N = 256 NI <= 2048, S <= 8. h may be NULL. */
int camx_q3p_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h,
                       uint16_t * h16, int N, int n, camx_stream_t stream);
/* q35p_add_rms16 (kernels/q35_prefill.hip:636-660) = the dense line's OP_OWN_ADD_RMS16 (kernels/k3_q35_ops.h:79-145).
 * x = x + d (d NULL: no add), any N = 256 NI <= 65536; h and h16 are both written. */
int camx_q35p_add_rms16(float * x, const float * d, const float * nw, float eps, float * h, uint16_t * h16, int N, int n,
                        camx_stream_t stream);
/* The same row pass with a q8_1 copy of h (36-byte blocks, [n][N / 32]): OP_RMS_MUL's optional q8_1 output
 * (kernels/k3_gguf_ops.h:1233-1268, q8_emit :158-162) on q3p_add_rms16's add. h, h16, q8 optional; N % 32 == 0. */
int camx_add_rms_q8_1(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h,
                      uint16_t * h16, void * q8, int N, int n, camx_stream_t stream);
/* Dense bf16 prefill form: x (fp32 residual) = x + bf16 addend d (kernels/core.hip:57-61's promotion; d NULL: no add), then
 * q35p_add_rms16's norm; hbf = bf16 copy of h by round-to-nearest-even (kernels/prefill_glue.hip:77-80). h, hbf optional. */
int camx_add_rms_bf16(float * x, const uint16_t * d, const float * nw, float eps, float * h, uint16_t * hbf, int N, int n,
                      camx_stream_t stream);
/* pf_rms_mul (kernels/prefill_glue.hip:94-124): y[r] = (x[r] * scale_r) * w[r % wr] for R rows of K values; y (may be x),
 * ybf (bf16 copy), scl (row scale [R]) each optional. The reference kernel is built for K = 2560; K is an argument here. */
int camx_pf_rms_mul(const float * x, const float * w, float * y, uint16_t * ybf, float * scl, int R, int wr, float eps, int K,
                    camx_stream_t stream);
/* OP_OWN_ADD_RMS16 (kernels/k3_own_ops.h:326-383) with the tape's Seg fields (python/caminus/engine/k3.py:881-902): y = x, a = d,
 * gs = w, pad1 = S, W = nw, rs = eps, asum = h, aux = h16, N, K = the token stride of h16 in elements (>= N), team = tokens.
 * camx_q3p_add_rms16 is the same pass with K = N. Rows longer than 2048 values exist only on the dense line's modules and are forwarded
 * to camx_op_q35_add_rms16 (S <= 1, w NULL, h required). */
int camx_op_own_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h, uint16_t * h16,
                          int N, int K, int tokens, camx_stream_t stream);
/* OP_OWN_ADD_RMS16 as the dense line's modules run it (kernels/k3_q35_ops.h:79-130, host python/caminus/engine/k3.py:881-902): any row length
 * N = 256 NI up to 65536, S = 1 (x += d) or 0, h always written, the fp16 copy rounded once from the last product (camx_q35p_add_rms16's
 * arithmetic) at token stride K. The reference selects this form by module; camx_op_own_add_rms16 forwards rows longer than 2048 here. */
int camx_op_q35_add_rms16(float * x, const float * d, int S, const float * nw, float eps, float * h, uint16_t * h16, int N, int K, int tokens,
                          camx_stream_t stream);
/* OP_GG_Q8_1 (kernels/k3_gguf_ops.h:55-77) with the tape's Seg fields in their order (python/caminus/engine/k3.py:649-659):
 * a = x, y, N = n, work = 0 plain / 1 silu(x * rs) / 2 silu(x) * gs[i], rs, gs. The same blocks as camx_gg_quantize_q8_1. */
int camx_op_gg_q8_1(const float * x, void * y, int n, int work, float rs, const float * gs, camx_stream_t stream);
/* OP_OWN_EMB (kernels/k3_own_ops.h:273-304) with the tape's Seg fields (python/caminus/engine/k3.py:904-921): W = the raw GGUF
 * table, a = tok, y = x fp32 [tokens][N], N = the row length D, K = row bytes, work = the format's GG number (4 Q4_K, 7 IQ2_S of
 * kernels/k3_q35t_ops.h:147-175; 3 Q8_0 is taken too), pad1 = 1: tok is the 64-bit key word of OP_OWN_ARGMAX and the token the
 * complement of its low half (tokens must be 1), pad2 = vocab (ids are clamped to [0, vocab)), ntask = tokens. The same rows as
 * camx_q3p_emb / camx_emb_gather. */
int camx_op_own_emb(const uint8_t * W, const void * tok, float * x, int N, int K, int work, int pad1, int pad2, int tokens,
                    camx_stream_t stream);
/* OP_GDN_CONV (kernels/k3_q35_ops.h:148-177) with the tape's Seg fields (python/caminus/engine/k3.py:993-1000): the decode / verify
 * form of the GDN short convolution with a lazy commit. W = w fp32 [C][4], gs = state fp32 [C][3], a = x fp32 [T][C], asum = the
 * pass parameters (int32; [1] = mprev, the previous pass's accepted tokens, clamped to [0, T]), y = out fp32 [T][C], aux = xprev
 * fp32 [T][C], N = C; T = the tape's tokens per pass. Per channel: the state first shifts in xprev[0 .. mprev) and is stored; then
 * out[t] = silu(state . w[0..2] + x[t] w[3]) along the T tokens without storing the state again, and xprev[t] = x[t]. */
int camx_op_gdn_conv(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, int C, int T,
                     camx_stream_t stream);
/* OP_RMS_MUL (kernels/k3_gguf_ops.h:1233-1268; Seg fields: a = x, W = w, y, asum = q8, N = R, K, pad1 = wr, rs = eps). */
int camx_op_rms_mul(const float * x, const float * w, float * y, void * q8, int R, int wr, int K, float eps, camx_stream_t stream);
/* The remaining hot-path ops of the decode tape by their Seg fields (python/caminus/engine/k3.py:393-399). The tape keeps its position in an
 * int32 word ON THE DEVICE (Seg.asum), so a captured graph advances by a device-side increment; these forms read it there.
 * OP_QK_NR (k3.py:1057-1063; kernels/k3_gguf_ops.h:1495-1518): a = x, pad1 = head_stride, W = w, asum = pos (row r at pos[0] + r / heads),
 * y = out, out_f32 = n_rot, rs = theta_scale, pad2 = eps_bits (the bit pattern of eps), N = T * heads, K = dim; fp32. */
int camx_op_qk_nr(const float * x, int head_stride, int heads, int dim, const float * w, const int32_t * pos, float * out, int n_rot,
                  float theta_scale, int eps_bits, int T, camx_stream_t stream);
/* OP_KV_APPEND (k3.py:1065-1089; kernels/k3_gguf_ops.h:1520-1553, kernels/k3_q35_kvq8_ops.h:16-27): a = k, W = v (fp32 [T][M]), y = cache,
 * asum = pos (token t to row pos[0] + t), N = M, gs = err. work 0: fp16 rows [K | V]; 1: ggml q8_0 rows; 2: the dense Q8 line's blocks with
 * the codec's refusal rules (the reference selects that form by its K3_Q35_KV_Q8 build, with work = 1 and its sticky word in gs). rows =
 * the cache's rows, checked on the device as the reference's launch guard does: err bit 1, the row is not written; bit 2 a refused block
 * (bytes untouched), bit 4 layout (work 2). */
int camx_op_kv_append(const float * k, const float * v, void * cache, const int32_t * pos, int M, int work, int * err, int rows, int T,
                      camx_stream_t stream);
/* OP_HADAMARD (k3.py:1244-1257): y = x in place, N = C chunks, K = n in {64, 128, 256}; rows_per_task is the tape's task size (ignored). */
int camx_op_hadamard(float * x, int C, int n, int rows_per_task, camx_stream_t stream);
/* OP_GATE_MUL16 (k3.py:1209-1219; kernels/k3_q35_ops.h:381-391): a, W = gate, y = out16 fp16, N = n, K = dim, pad1 = head_stride, pad2 = offset. */
int camx_op_gate_mul16(const float * a, const float * gate, int head_stride, int offset, uint16_t * out16, int n, int dim, camx_stream_t stream);
/* The dense Q8 line's OP_HADAMARD on the attention output and the OP_GATE_MUL16 behind it in one launch (python/caminus/engine/q35_dense.py:419-420):
 * chunks of hn in {64, 128, 256} values of a are transformed, then multiplied by the gate as above; a_out (optional, may be a) receives the
 * transformed values. dim % hn == 0, n % dim == 0, head_stride and offset multiples of 4, 16-byte aligned a / gate. Every bit equals
 * camx_op_hadamard followed by camx_op_gate_mul16. */
int camx_op_hadamard_gate_mul16(const float * a, float * a_out, const float * gate, int head_stride, int offset, uint16_t * out16, int n, int dim,
                                int hn, camx_stream_t stream);
/* OP_GDN_L2 (k3.py:1002-1008; kernels/k3_q35_ops.h:181-194): a = x, y = out, rs = eps / dim, N = T * heads, K = dim, pad1 = x_stride (0: heads * dim). */
int camx_op_gdn_l2(const float * x, float * out, int heads, int dim, float rs, int x_stride, int T, camx_stream_t stream);
/* OP_OWN_SWIGLU16 (k3.py:854-860; kernels/k3_own_ops.h:258-262): a = g, W = u, y = y16, N = n. */
int camx_op_own_swiglu16(const float * g, const float * u, uint16_t * y16, int n, camx_stream_t stream);
/* The tape's row ops on either side of the ones above, by their Seg fields; the arithmetic is that of the prefill kernels of the same names.
 * OP_OWN_F16 (k3.py:846-852; kernels/k3_own_ops.h:247-252): out16 = fp16(x), round to nearest even. */
int camx_op_own_f16(const float * x, uint16_t * out16, int n, camx_stream_t stream);
/* OP_OWN_MOE_SUM (k3.py:862-868; kernels/k3_own_ops.h:255-256, 263-271): x[i] += acc with acc = 0, then per slot fma(w[s], d[s * n + i], acc),
 * or acc + d[s * n + i] when w is NULL (the attention's residual add with slots = 1). slots 1 .. 64. */
int camx_op_own_moe_sum(const float * d, const float * w, float * x, int n, int slots, camx_stream_t stream);
/* OP_SHEXP_ADD (k3.py:958-963; kernels/k3_gguf_ops.h:1218-1229): out = moe + shexp * sigmoid(gate_logit[token]), n = T * (n / T) values. */
int camx_op_shexp_add(const float * moe, const float * shexp, const float * gate_logit, float * out, int n, int T, camx_stream_t stream);
/* OP_ADD_SUM (k3.py:1237-1242; kernels/k3_gguf_ops.h:1683-1692): y = y + (a + b). */
int camx_op_add_sum(const float * a, const float * b, float * y, int n, camx_stream_t stream);
/* OP_GDN_GATES (k3.py:1010-1015; kernels/k3_gguf_ops.h:1356-1372, kernels/k3_q35_ops.h:196-211): out [T][2H] = softplus(alpha + dt) * a |
 * sigmoid(beta); alpha, beta [T][H]. */
int camx_op_gdn_gates(const float * alpha, const float * beta, const float * dt, const float * a, float * out, int H, int T, camx_stream_t stream);
/* OP_GDN_NORM (k3.py:1037-1043; kernels/k3_gguf_ops.h:1461-1489): N = T * H heads of K values, out = ((o * rsqrt(mean(o^2) + eps)) * w) *
 * sigmoid(z), or * silu(z) with silu = 1 (the reference's K3_GDN_SILU builds); q8 (optional, K % 32 == 0) receives the q8_1 blocks of out
 * (a second launch). K % 4 == 0, K <= 1024, 16-byte aligned rows, as camx_pf_gdn_norm. */
int camx_op_gdn_norm(const float * o, const float * w, const float * z, float * out, void * q8, int N, int K, float eps, int silu,
                     camx_stream_t stream);
/* OP_GDN_NORM16 (k3.py:1045-1055; kernels/k3_q35_ops.h:314-333): the SiLU form with fp16 output. */
int camx_op_gdn_norm16(const float * o, const float * w, const float * z, uint16_t * out16, int N, int K, float eps, camx_stream_t stream);
/* OP_GATE_MUL (k3.py:1201-1207; kernels/k3_gguf_ops.h:1607-1619): out fp32 = a * sigmoid(gate[(i / dim) * head_stride + offset + i % dim]);
 * q8 (optional, n % 32 == 0) receives the q8_1 blocks of out (a second launch). */
int camx_op_gate_mul(const float * a, const float * gate, int head_stride, int offset, float * out, void * q8, int n, int dim,
                     camx_stream_t stream);
/* The prologue of OP_OWN_ATTS (k3.py:1151-1199, Seg.asum = pos; kernels/k3_own_atts.h:183-274): camx_q3p_qk_rope / _q8 with token t at
 * pos[0] + t read on the device, checked there against the cache's `rows` (err bit 1: the row is not written, q16 is). err is required. */
int camx_op_own_qk_rope(const float * qkv, int ldq, int nh, int nkv, const float * par, const int32_t * pos, uint16_t * q16, void * cache,
                        int rows, int * err, int n, int yarn, int q8, camx_stream_t stream);
/* OP_GDN_CONV followed by OP_GDN_L2, the pair the tape appends back to back (python/caminus/engine/q35_dense.py:399-400), in one launch:
 * camx_op_gdn_conv's arguments, then qk [T][heads][128] = camx_op_gdn_l2(y, qk, heads, 128, rs, C, T). Same bits as the two. C % 128 == 0. */
int camx_op_gdn_conv_l2(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, float * qk, int C,
                        int T, int heads, float rs, camx_stream_t stream);
/* OP_GDN_GATES, OP_GDN_CONV and OP_GDN_L2, the three row ops a linear-attention layer of the tape runs ahead of its recurrence
 * (python/caminus/engine/q35_dense.py:396-400), in one launch: camx_op_gdn_conv_l2's arguments, then camx_op_gdn_gates' (alpha, beta [T][H],
 * gates [T][2H]). Same bits as the two calls. */
int camx_op_gdn_conv_l2_gates(const float * w, float * state, const float * x, const int32_t * params, float * y, float * xprev, float * qk, int C,
                              int T, int heads, float rs, const float * alpha, const float * beta, const float * dt, const float * a, float * gates,
                              int H, camx_stream_t stream);
/* pf_hc_post_rms (kernels/prefill_glue.hip:130-170): row q = t * HC + h of N values: res[q] = fma(b[t], 2 sigmoid(inj[q] * rs),
 * res[q]) in place, then the norm of the updated row with w[h]: xn fp32, xnbf bf16, scl the row scale [T * HC], each optional.
 * The reference kernel is built for N = 2560; N is an argument here. */
int camx_pf_hc_post_rms(const float * b, const float * inj, float * res, const float * w, float * xn, uint16_t * xnbf, float * scl,
                        int T, int HC, float rs, float eps, int N, camx_stream_t stream);
/* pf_hc_post (kernels/prefill_glue.hip:172-188): the residual update alone. */
int camx_pf_hc_post(const float * b, const float * inj, float * res, int T, int HC, int D, float rs, camx_stream_t stream);
/* pf_hc_mean (kernels/prefill_glue.hip:190-206): out[t][i] = rs * sum over h of xn[t][h][i] * sigmoid(g[t][h][i]) (fma chain from
 * 0); xn = x, or (scl and w given) recomputed from the residual x as (x * scl[t * HC + h]) * w[h][i]. */
int camx_pf_hc_mean(const float * x, const float * scl, const float * w, const float * g, float * out, int T, int HC, int D, float rs,
                    camx_stream_t stream);
/* rmsnorm_f32 (kernels/core.hip:30-46): out = x * inv * w over `rows` rows of D values (any D). */
int camx_rmsnorm_f32(const float * x, const float * w, float * out, int D, float eps, int rows, camx_stream_t stream);

/* ---- q8_1 activation quantizers ------------------------------------------------------------------------------------------ */
/* gg_quantize_q8_1 (kernels/k3_gguf.hip:29-36) and OP_GG_Q8_1 (kernels/k3_gguf_ops.h:55-77): y = ceil(n / 32) blocks of
 * {half d, half sum, int8 qs[32]}; mode 0 plain, 1 silu(x * rs), 2 silu(x) * g[i]; values past n quantize as 0. */
int camx_gg_quantize_q8_1(const float * x, void * y, long n, int mode, float rs, const float * g, camx_stream_t stream);
/* quantize_mmq_q8_1<layout, false> (kernels/ggml_mmq/quantize_mmq.cuh:41-140; launched by prefill/mmq.py:245-261):
 * column c of vy = row (ids ? ids[c] : c) of x (row stride s01 floats), blocks of 144 bytes per 128 values in
 * [ne0 / 128][ne1] order, ne00 = K, ne0 = K padded to 512 (padding quantizes as zeros). layout 0 = D4, 1 = DS4.
 * s02, s03 must be 0 and ne2 1 (the reference's callers pass exactly that). */
int camx_quantize_mmq_q8_1(const float * x, const int32_t * ids, void * vy, long ne00, long s01, long s02, long s03, long ne0,
                           int ne1, int ne2, int n_expert_used, int layout, camx_stream_t stream);
/* quantize_mmq_q8_1<layout, true> (same source; prefill/mmq.py:263-276): token t's row (stride s02 floats) quantized once and
 * written to the columns ids[t * n_expert_used + slot] of the ne1 = ntok * n_expert_used compact columns. */
int camx_quantize_mmq_q8_1_scatter(const float * x, const int32_t * ids, void * vy, long ne00, long s01, long s02, long s03,
                                   long ne0, int ne1, int ne2, int n_expert_used, int layout, int ntok, camx_stream_t stream);
/* Fused SwiGLU -> MMQ q8_1: gu bf16 [T][ld] = [g (F) | u (F)]; act = bf16(bf16(silu g) * u) (silu_mul_bf16,
 * kernels/core.hip:48-55) quantized as quantize_mmq_q8_1 of the fp32-widened act. act (optional, bf16 [T][F]) receives
 * the activation. Fills the per-device lookup tables on its first call (synchronizes `stream` once). Every input gives
 * camx_silu_mul_bf16's bits: a NaN in the activation (a NaN or infinite input) is stored as the canonical 0x7fc0 that f2bf
 * (kernels/core.hip:14-21) writes, and the block sums are taken from that value. */
int camx_swiglu_mmq_q8_1(const uint16_t * gu, long ld, long F, void * vy, uint16_t * act, int T, int layout, camx_stream_t stream);

/* ---- SwiGLU, gates ------------------------------------------------------------------------------------------------------------ */
/* q3p_swiglu (kernels/q3m_prefill.hip:516-518) = OP_OWN_SWIGLU16 (kernels/k3_own_ops.h:258-262): y16 = fp16(silu(g) * u). */
int camx_q3p_swiglu(const float * g, const float * u, uint16_t * y16, int n, camx_stream_t stream);
/* gg_silu_mul (kernels/k3_gguf.hip:74-77): h = silu(g) * u in fp32. */
int camx_gg_silu_mul(const float * g, const float * u, float * h, int n, camx_stream_t stream);
/* silu_mul_bf16 (kernels/core.hip:48-55): act[r][c] = bf16(bf16(silu(g)) * u), gu rows = [g (H) | u (H)], n = rows * H. */
int camx_silu_mul_bf16(const uint16_t * gu, uint16_t * act, int H, long n, camx_stream_t stream);
/* pf_gate_mul (kernels/prefill_attn.hip:379-386; io 0: fp32 -> fp32), q35p_gate_mul16 / OP_GATE_MUL16
 * (kernels/q35_prefill.hip:960-969, kernels/k3_q35_ops.h:381-391; io 1: fp32 -> fp16), io 2: bf16 a and gate -> bf16:
 * y[i] = a[i] * sigmoid(gate[(i / D) * stride + off + i % D]) over N elements. */
int camx_gate_mul(const void * a, const void * gate, void * y, long N, int D, int stride, int off, int io, camx_stream_t stream);

/* ---- QK-norm + rotary, KV rows ------------------------------------------------------------------------------------------------ */
/* q3p_qk_rope (kernels/q3m_prefill.hip:534-591, F16 form; yarn = the Q3P_YARN build): n tokens at positions pos0 + t;
 * qkv fp32 [n][ldq] = q (nh heads of 128) | k (nkv) | v (nkv); par = q_norm[128] | k_norm[128] | theta_scale | eps
 * (| freq[64] | mscale when yarn); q16 fp16 [n][nh][128]; cache = fp16 rows [K | V] indexed by position. The caller has
 * checked the positions against the cache's rows (prefill/q3m_ops.py:103-117); pos0 < 0 (or pos0 + n past INT_MAX) is refused here (1), for
 * this and the next two entry points. */
int camx_q3p_qk_rope(const float * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint16_t * cache,
                     int n, int yarn, camx_stream_t stream);
/* q3p_qk_rope_q8 (same source under Q3P_KV_Q8; rotation kernels/own_kv_rot128.h:21-33, block encode
 * kernels/own_kv_codec.h:57-72): K = Hadamard-128 of the fp16-rounded rotary output, V = fp16-rounded v, both as Q8 blocks;
 * q16 = fp16 of the same transform of q. err: bit 2 ORed when a block is refused (its bytes stay untouched). */
int camx_q3p_qk_rope_q8(const float * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint8_t * cache,
                        int * err, int n, int yarn, camx_stream_t stream);
/* The same statements on bf16 activations (qkv bf16, widened exactly), F16 rows: a dense bf16 prefill chunk. */
int camx_qk_rope_bf16(const uint16_t * qkv, int ldq, int nh, int nkv, const float * par, int pos0, uint16_t * q16, uint16_t * cache,
                      int n, int yarn, camx_stream_t stream);
/* Batched decode form of the two kernels above: sequence t at its own position pos[t]; with page_table the row address is
 * (page_table[t * pt_stride + pos / page] * page + pos % page) * row_bytes, else pos * row_bytes. q8 selects the row format.
 * With page_table NULL, n_pages is the number of rows of the cache. err (required) bit 1: a position outside the sequence's
 * table row (pos < 0 or pos / page >= pt_stride) or outside the unpaged cache; bit 8: a page id outside [0, n_pages). Either way
 * that sequence's row is not written (q16 is). Paging has no reference counterpart: each row's bytes equal the unpaged kernel's. */
int camx_qk_rope_paged(const float * qkv, int ldq, int nh, int nkv, const float * par, const int32_t * pos, uint16_t * q16,
                       void * cache, int * err, const int32_t * page_table, int pt_stride, int page, int n_pages, int n, int yarn,
                       int q8, camx_stream_t stream);
/* pf_qk_nr (kernels/prefill_attn.hip:106-129) = OP_QK_NR (kernels/k3_gguf_ops.h:1495-1518, kernels/k3_q35_ops.h:341-364):
 * out [T][heads][D] = rotary on the first nrot dims of rms_norm(x head) * w, row r at position pos0 + r; input heads sit
 * head_stride elements apart; D <= 512. io 0: fp32 in / out, 1: bf16 in / out. */
int camx_pf_qk_nr(const void * xin, int head_stride, int heads, const float * w, int D, int nrot, float theta_scale, float eps,
                  int pos0, void * out, int T, int io, camx_stream_t stream);
/* The same with one position per row (a speculative-verify batch). */
int camx_qk_nr_pos(const void * xin, int head_stride, int heads, const float * w, int D, int nrot, float theta_scale, float eps,
                   const int32_t * pos, void * out, int T, int io, camx_stream_t stream);
/* The q heads and the k heads of a token in one launch (the two OP_QK_NR segments of a full-attention layer,
 * python/caminus/engine/q35_dense.py:408-415): nh heads at xq + (t * nh + h) * q_stride with weight wq -> outq [T][nh][D], nkv heads at
 * xk + (t * nkv + h) * k_stride with wk -> outk [T][nkv][D]. Row t sits at pos[t] (pos given), else pos_dev[0] + t (pos_dev given: a
 * device word), else pos0 + t. The same bits as two camx_pf_qk_nr / camx_qk_nr_pos calls (and, from T * nh >= 12288, their two launches). */
int camx_qk_nr_qk(const void * xq, int q_stride, int nh, const float * wq, const void * xk, int k_stride, int nkv, const float * wk, int D,
                  int nrot, float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, void * outq, void * outk,
                  int T, int io, camx_stream_t stream);
/* The fp16 and q8_0 cache lines' chain in one launch (python/caminus/engine/q3moe_one.py:316-318 and 368-370, the non-Q8 branch of
 * python/caminus/engine/q35_dense.py:408-415: OP_QK_NR k -> OP_KV_APPEND, and OP_QK_NR q; kernels/k3_gguf_ops.h:1520-1553): q and k heads,
 * weights and positions as camx_qk_nr_qk, fp32; v [T][nkv * D] at ldv; qo [T][nh][D]; ko [T][nkv][D] or NULL (the normed k then reaches
 * only the cache); cache row position(t): work 0 fp16 [K | V], work 1 ggml q8_0 blocks of K then of V (D % 32 == 0). err bit 1: a position
 * outside [0, rows), that cache row is not written (qo and ko are). D % 4 == 0, strides % 4 == 0, fp32 pointers 16-byte aligned, else
 * CAMX_EINVAL. Every byte equals camx_qk_nr_qk followed by camx_op_kv_append on its k output. One launch of a wave per head, meant for decode
 * and verify batches; from T * nh >= 12288 with ko given (and no position array) it runs the prefill-sized kernels of the three ops instead. */
int camx_qk_nr_kv(const float * q, int q_stride, int nh, const float * wq, const float * k, int k_stride, const float * v, int ldv, int nkv,
                  const float * wk, int D, int nrot, float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, float * qo,
                  float * ko, void * cache, int work, int rows, int * err, int T, camx_stream_t stream);
/* The dense Q8 line's per-token chain in one launch (python/caminus/engine/q35_dense.py:409-418: OP_QK_NR k -> OP_HADAMARD 256 ->
 * OP_HADAMARD 64 on v -> OP_KV_APPEND with kernels/k3_q35_kvq8_ops.h:16-27's Q8 writer, and OP_QK_NR q -> OP_HADAMARD 256): heads of 256
 * dims, fp32. q [T][nh] heads at q_stride floats (the q | gate interleave), k and v [T][nkv * 256] at ldk / ldv; qo [T][nh][256] = the
 * transformed q; cache row (position) = Q8 blocks of the transformed k heads | Q8 blocks of H64(v). Positions as in camx_qk_nr_qk. err bits:
 * 1 a position outside [0, rows) (row not written; qo is), 2 a refused block (its bytes stay). nrot in {16, 32, 64, 128, 256}. Every byte
 * equals camx_pf_qk_nr + camx_pf_hadamard + camx_own_kv_q8_append on the same inputs. */
int camx_qk_nr_q8(const float * q, int q_stride, int nh, const float * k, int ldk, const float * v, int ldv, int nkv, const float * qn,
                  const float * kn, int nrot, float theta_scale, float eps, int pos0, const int32_t * pos_dev, const int32_t * pos, float * qo,
                  uint8_t * cache, int rows, int * err, int T, camx_stream_t stream);
/* out[j] = the frequency of rotary pair j as the kernels above compute it: the correctly rounded theta_scale ** j. */
int camx_rope_freqs(float theta_scale, int n, float * out, camx_stream_t stream);

/* own_kv_q8_append (kernels/kv_codec.hip:10-30 with kernels/own_kv_codec.h:33-52; launcher device/kv_codec.py:48-83):
 * T rows of M values from k / v (row strides ldk / ldv) to cache rows pos0 + t of 2 * (M / 32) blocks of 34 bytes.
 * err bits: 1 position outside [0, rows), 2 refused block (bytes untouched), 4 layout (M < 32, M % 32, ld < M, rows < 1). */
int camx_own_kv_q8_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, int rows,
                          int * err, int T, camx_stream_t stream);
/* The reader of those rows. The reference has no kernel of its own for it: its attention kernels decode blocks in place
 * (q3p_q8_stage, kernels/q3m_prefill.hip:617-632; host reference decode_q8_kv, python/caminus/ref_kv.py:127-144). Row t =
 * row_ids ? row_ids[t] : pos0 + t; value = (float)code * (float)half scale; k, v [T][ld] fp32 (f16 = 0) or fp16 bits rounded
 * from that value (f16 = 1, the prefill staging's operand format). err bits: 1 a row outside [0, rows) (outputs untouched), 4
 * layout. */
int camx_own_kv_q8_read(const uint8_t * cache, const int32_t * row_ids, int pos0, int rows, int M, void * k, int ldk, void * v, int ldv,
                        int * err, int T, int f16, camx_stream_t stream);
/* pf_kv_append, q8_0 rows (kernels/prefill_attn.hip:157-181) = OP_KV_APPEND work 1 (kernels/k3_gguf_ops.h:1532-1553):
 * no refusal rules; err bit 1 for a row outside [0, rows). */
int camx_pf_kv_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, int rows, int * err,
                      int T, camx_stream_t stream);
/* pf_hadamard (kernels/prefill_attn.hip:132-153) = OP_HADAMARD (kernels/k3_gguf_ops.h:1699-1721): in place, C chunks of
 * n in {64, 128, 256} values, scale 1 / sqrtf(n). rpb (the reference's chunks per workgroup) is accepted and ignored. */
int camx_pf_hadamard(float * x, int C, int n, int rpb, camx_stream_t stream);
/* own_kv_rot128 as a kernel of its own (kernels/own_kv_rot128.h:21-33; CPU reference python/caminus/ref_kv.py:72-89):
 * y = H128 x per head of 128 values, scale 0x1.6a09e6p-4f. */
int camx_hadamard128(const float * x, float * y, long heads, camx_stream_t stream);

/* ---- quantized embedding rows ------------------------------------------------------------------------------------------------ */
/* q3p_emb (kernels/q3m_prefill.hip:364-380) = OP_OWN_EMB (kernels/k3_own_ops.h:279-304): x [n][N] fp32 = the Q4_K rows
 * toks[i] of W (rb bytes per row), ids clamped to [0, vocab). */
int camx_q3p_emb(const uint8_t * W, int rb, int vocab, const int32_t * toks, float * x, int N, int n, camx_stream_t stream);
/* Gather + dequant to fp32 (x) and / or bf16 (xbf); fmt 0 = Q4_K (as q3p_emb), 1 = Q8_0 (the host decoder's arithmetic,
 * python/caminus/own_dequant.py:202-206), 2 = IQ4_XS (as embd_rows_iq4xs), 3 = IQ2_S (q35t_op_emb's rows,
 * kernels/k3_q35t_ops.h:147-175; python/caminus/own_dequant.py:128-137). N = 256 NI <= 8192. W and rb aligned to 16 / 2 / 8 / 2. */
int camx_emb_gather(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n, int fmt,
                    camx_stream_t stream);
/* Gather + dequant + (x += d) + RMSNorm * nw with fp32 / fp16 / q8_1 copies of the normed row in one pass per row
 * (q3p_emb followed by q3p_add_rms16 and OP_RMS_MUL's q8_1 copy). xbf = bf16 of the gathered row; x = the residual row. The addend d must
 * not overlap x (up to 256 rows a row's slabs are written by four waves that each read the whole addend row). */
int camx_emb_gather_add_rms(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, const float * d,
                            const float * nw, float eps, float * h, uint16_t * h16, void * q8, int N, int n, int fmt,
                            camx_stream_t stream);

/* embd_rows_iq4xs (kernels/prefill_feed.hip:40-54): out [n][256 nblk] fp32 = the IQ4_XS rows tok[i] of table ([nvocab][136 nblk]);
 * an id outside [0, nvocab) is clamped and reported as bit 1 (value 2) of *err. */
int camx_embd_rows_iq4xs(const uint8_t * table, const int32_t * tok, int nvocab, int n, int nblk, float * out, int * err,
                         camx_stream_t stream);
/* ple_rows_iq4nl (kernels/prefill_feed.hip:24-35): out [nrows][32 bpr] fp32 = the IQ4_NL rows inv[r] of raw ([nuniq][18 bpr]);
 * an index outside [0, nuniq) is clamped and reported as bit 0 (value 1) of *err. */
int camx_ple_rows_iq4nl(const uint8_t * raw, const int32_t * inv, int nuniq, int nrows, int bpr, float * out, int * err,
                        camx_stream_t stream);

/* ---- GDN short convolution and L2 norm ------------------------------------------------------------------------------------------ */
/* pf_gdn_conv (kernels/prefill_glue.hip:314-332) = OP_GDN_CONV (kernels/k3_q35_ops.h:152-177): y[t][c] = silu(fma chain
 * of [x(t-3) .. x(t)] . w[c]), times before 0 from state[c] = [x(-3), x(-2), x(-1)]. bf16 != 0: x and y are bf16. */
int camx_pf_gdn_conv(const void * x, const float * w, const float * state, void * y, int C, int T, int ldx, int ldy, int bf16,
                     camx_stream_t stream);
/* pf_conv_state (kernels/prefill_glue.hip:334-341): state[c] = the last 3 inputs of [state[c], x[0 .. T-1][c]]. */
int camx_pf_conv_state(const void * x, float * state, int C, int T, int ldx, int bf16, camx_stream_t stream);
/* pf_gdn_l2 (kernels/prefill_gdn.hip:66-78) = OP_GDN_L2 (kernels/k3_q35_ops.h:181-194): per head of K <= 512 values
 * y = (scale * x) * (1 / sqrt(K)), scale = 1 / sqrt(sum x^2 / K + rs); head h of token t at x + t * ldx + h * K. */
int camx_pf_gdn_l2(const void * x, void * y, int heads, int K, int ldx, float rs, int T, int bf16, camx_stream_t stream);
/* pf_gdn_conv and pf_gdn_l2 in one launch (the reference runs them back to back: python/caminus/engine/q35_dense.py:399-400,
 * kernels/k3_q35_ops.h:152-194): y (optional) = camx_pf_gdn_conv's rows; qk [T][heads][128] = camx_pf_gdn_l2(y, heads, 128, ldy, rs), the
 * norm of the first heads * 128 channels, taken from the values as y stores them. Same bits as the two calls. C % 128 == 0, operands
 * 16-byte aligned, ldx / ldy multiples of 4 (fp32) or 8 (bf16). The state is read only (camx_pf_conv_state advances it). */
int camx_gdn_conv_l2(const void * x, const float * w, const float * state, void * y, void * qk, int C, int T, int ldx, int ldy, int heads,
                     float rs, int bf16, camx_stream_t stream);

/* ---- S1 core and fused residual (kernels/core.hip, kernels/fuse.hip) ------------------------------------------------------------- */
int camx_embedding_f32(const int * tok, const float * emb, float * out, int D, int T, camx_stream_t stream);          /* core.hip:23-28 */
int camx_residual3(const float * x, const uint16_t * m, const uint16_t * y, float * out, long n, camx_stream_t stream); /* core.hip:57-61 */
int camx_cast_bf16(const float * x, uint16_t * out, long n, camx_stream_t stream);                                     /* core.hip:63-66 */
int camx_copy_cols_bf16(const uint16_t * in, int ld_in, int c_in, uint16_t * out, int ld_out, int c_out, int n, long rows,
                        camx_stream_t stream);                                                                          /* core.hip:69-75 */
/* residual_slices_fwd (kernels/fuse.hip:19-33): out = ((x + m) + mlp) + (pos[r] >= 0 ? ys[pos[r]] : 0); ys / pos may be NULL. */
int camx_residual_slices_fwd(const float * x, const uint16_t * m, const uint16_t * mlp, const uint16_t * ys, const int * pos,
                             float * out, int d, long n4, camx_stream_t stream);

/* residual_slices_bwd (kernels/fuse.hip:35-47): dm = dmlp = bf16(dout); dys[pos[r]] = bf16(dout[r]) where pos[r] >= 0 (dx = dout is
 * the caller's). pos / dys may be NULL. */
int camx_residual_slices_bwd(const float * dout, const int * pos, uint16_t * dm, uint16_t * dmlp, uint16_t * dys, int d, long n4,
                             camx_stream_t stream);

/* ---- more row kernels of the batched prefill ------------------------------------------------------------------------------------------ */
/* pf_gdn_norm (kernels/prefill_gdn.hip:385-407): per (token, value head) row of K values, y = ((o * rsqrt(mean(o^2) + eps)) * w) *
 * sigmoid(z) (silu = 0) or * silu(z) (silu = 1: the reference's PF_GDN_SILU build). K % 4 == 0, K <= 1024. */
int camx_pf_gdn_norm(const float * o, const float * w, const float * z, float * y, int K, float eps, long rows, int silu, camx_stream_t stream);
/* q35p_gdn_norm16 (kernels/q35_prefill.hip:671-692): the silu form with fp16 output. */
int camx_q35p_gdn_norm16(const float * o, const float * w, const float * z, uint16_t * y16, int K, float eps, long rows, camx_stream_t stream);
/* pf_gdn_gates (kernels/prefill_gdn.hip:80-92): y [T][2H] = softplus(alpha + dt) * a | sigmoid(beta); alpha / beta rows at lda / ldb. */
int camx_pf_gdn_gates(const float * alpha, int lda, const float * beta, int ldb, const float * dt, const float * a, float * y, int H, int T,
                      camx_stream_t stream);
/* q35p_kv_append16 (kernels/q35_prefill.hip:694-707): cache[pos0 + t] = fp16(k[t]) | fp16(v[t]) (2 M halves per position); a row at
 * or past `rows` is not written and sets bit 0 of *err. */
int camx_q35p_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, int rows, int * err, int T,
                          camx_stream_t stream);
/* pf_add_sum (kernels/prefill_glue.hip:416-423): y = y + (a + b). */
int camx_pf_add_sum(const float * a, const float * b, float * y, long n, camx_stream_t stream);
/* pf_silu_bf16 / pf_to_bf16 (kernels/prefill_glue.hip:552-566): y [Tpad][K] = bf16(silu(fma(rs, x, 0))) / bf16(x) for rows < T (x rows
 * at ldx), zero rows from T to Tpad. */
int camx_pf_silu_bf16(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, float rs, camx_stream_t stream);
int camx_pf_to_bf16(const float * x, int ldx, uint16_t * y, int T, int Tpad, int K, camx_stream_t stream);
/* pf_hc_avg (kernels/prefill_attn.hip:388-397): y[t][i] = (((r0 + r1) + r2) + ..) * (1 / hc) of r [T][hc][D]; y rows at ldo. */
int camx_pf_hc_avg(const float * r, float * y, int T, int hc, int D, int ldo, camx_stream_t stream);
/* pf_ple_gate (kernels/prefill_glue.hip:343-372): per token and stream, gate = sigmoid(sgn(s) sqrt(max(|s|, 1e-6))), s = (kn . qn) /
 * sqrt(D); gated = val * gate. qn = q, or (q * qscl) * qw when qscl / qw are given. gated may alias kn. HC <= 8. */
int camx_pf_ple_gate(const float * kn, const float * q, const float * qscl, const float * qw, const float * val, int ldv, float * gated,
                     float * gate_out, int HC, int D, int T, camx_stream_t stream);
/* pf_ple_conv / pf_ple_hist (kernels/prefill_glue.hip:374-414): dilated 4-tap conv with fp16 weights + silu over a chunk, optionally
 * fused with res = res + (a + conv); the history of the last 3 dil inputs per channel (3 dil <= 32). */
int camx_pf_ple_conv(const float * x, const float * xscl, const float * xw, const uint16_t * w, const float * hist, float * y, const float * a,
                     float * res, int C, int T, int D, int dil, camx_stream_t stream);
int camx_pf_ple_hist(const float * x, const float * xscl, const float * xw, float * hist, int C, int T, int D, int dil, camx_stream_t stream);

/* ---- activation fake-quant, forward (kernels/actq.hip) ------------------------------------------------------------------------------ */
/* actq_fwd_{f32,bf16} and actq_fwd_codes_{f32,bf16} (kernels/actq.hip:96-132, 315-326): M rows of K values (K % 128 == 0,
 * K <= 8192); y bf16 [M][K] (optional when codes are written), s [M] (optional), codes [M][K / 2] bytes (optional). */
int camx_actq_fwd(const void * x, int is_bf16, uint16_t * y, float * s, uint16_t * codes, int K, float clip, int qmax, int M,
                  camx_stream_t stream);
/* silu_mul_actq_fwd (kernels/actq.hip:307-310): the source is bf16(bf16(silu g) * u) of gu rows (stride ld) = [g (F) | u (F)]. */
int camx_silu_mul_actq_fwd(const uint16_t * gu, int ld, int F, uint16_t * y, float * s, uint16_t * codes, float clip, int qmax, int M,
                           camx_stream_t stream);
/* block_entry_fwd (kernels/actq.hip:247-274): RMSNorm(x) never materialized -> actq -> nab gate projections. */
int camx_block_entry_fwd(const float * x, const float * nw, const uint16_t * wab, int nab, float eps, uint16_t * y, float * s,
                         uint16_t * codes, uint16_t * ab, float * rstd_out, int d, float clip, int qmax, int M, camx_stream_t stream);

/* ---- activation fake-quant, backward (kernels/actq.hip) ----------------------------------------------------------------------------- */
/* actq_bwd_{f32,bf16} (kernels/actq.hip:158-218, 327-333): x the forward's input, g bf16 [M][K] the gradient of y; dx [M][K] in
 * x's type. Straight-through mask strictly inside the code range; the scale's gradient flows to the row's max-|u| elements. */
int camx_actq_bwd(const void * x, int is_bf16, const uint16_t * g, void * dx, int K, float clip, int qmax, int M, camx_stream_t stream);
/* silu_mul_actq_bwd (kernels/actq.hip:137-153, 311-314): dgu bf16 [M][2F] = [dg | du], contiguous rows. */
int camx_silu_mul_actq_bwd(const uint16_t * gu, int ld, int F, const uint16_t * g, uint16_t * dgu, float clip, int qmax, int M,
                           camx_stream_t stream);
/* block_entry_bwd (kernels/actq.hip:275-304): rstd [M] as the forward wrote it; dy bf16 [M][d]; dab bf16 [M][nab] (nab even; rows
 * [0, nab / 2) and [nab / 2, nab) of wab are two projections); dx fp32 [M][d]; d <= 1024. x, nw and dx 16-byte aligned, dy and wab
 * 8-byte aligned. */
int camx_block_entry_bwd(const float * x, const float * nw, const float * rstd, const uint16_t * wab, int nab, const uint16_t * dy,
                         const uint16_t * dab, float * dx, int d, float clip, int qmax, int M, camx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CAMX_H */
