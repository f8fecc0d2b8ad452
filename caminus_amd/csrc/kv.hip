// Q8 KV wire codec and Walsh-Hadamard transforms for gfx950. Replaces own_kv_q8_append (kernels/kv_codec.hip:10-30 with
// kernels/own_kv_codec.h:33-52), pf_kv_append's q8_0 rows (kernels/prefill_attn.hip:157-181) and pf_hadamard /
// OP_HADAMARD (kernels/prefill_attn.hip:132-153, kernels/k3_gguf_ops.h:1699-1721).
//
// A row is [K blocks | V blocks], 34 bytes per 32 values (fp16 scale + 32 int8). 8 lanes x 4 values encode one block; a
// wave encodes 8 blocks per step. Blocks are only 2-byte aligned, so codes go out as 16-bit stores and a refused block
// keeps every one of its bytes.
#include "common.cuh"

typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// Error bits: 1 position span, 2 numerical domain, 4 layout.
__global__ void __launch_bounds__(256) kv_q8_append_rows(const float * __restrict__ k, int ldk, const float * __restrict__ v, int ldv, int M,
                                                         uint8_t * __restrict__ cache, int pos0, int rows, int * __restrict__ err,
                                                         const int32_t * __restrict__ posb = nullptr) {
    if (M < 32 || M % 32 || ldk < M || ldv < M || rows < 1) {
        if (threadIdx.x == 0) atomicOr(err, 4);
        return;
    }
    if (posb) pos0 = posb[0];                            // the tape's device-resident position
    const long pos = (long)pos0 + (long)blockIdx.x;      // widened before the sum: a bad position cannot wrap into a valid row
    if (pos < 0 || pos >= rows) {
        if (threadIdx.x == 0) atomicOr(err, 1);
        return;
    }
    const size_t tt = blockIdx.x;
    const int nb = M / 32, lane = slot_of(threadIdx.x & 63), sub = lane & 7;
    uint8_t * dst = cache + (size_t)pos * ((size_t)2 * nb * 34);
    for (int b0 = (threadIdx.x >> 6) * 8; b0 < 2 * nb; b0 += 32) {
        const int b = b0 + (lane >> 3);
        const bool active = b < 2 * nb;
        const int bb = active ? b : 0;
        const float * x = (bb < nb ? k + tt * ldk : v + tt * ldv) + (size_t)(bb % nb) * 32 + 4 * sub;
        const f32x4 xv = *(const f32x4_a4 *)x;
        kv_q8_emit(xv, dst + (size_t)bb * 34, sub, err, active);
    }
}

// The same rows for a chunk of tokens with at most 32 blocks per row (M <= 512, 16-byte aligned): a wave per row, its (up to) four
// loads per lane issued together, four rows per workgroup. A workgroup per row is 4 KB of work; at chunk sizes the launch of 16384 such
// workgroups, not the memory, sets the time.
__global__ void __launch_bounds__(256) kv_q8_append_wave_rows(const float * __restrict__ k, int ldk, const float * __restrict__ v, int ldv, int M,
                                                              uint8_t * __restrict__ cache, int pos0, int rows, int T, int * __restrict__ err,
                                                              const int32_t * __restrict__ posb = nullptr) {
    const int tt = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tt >= T) return;
    if (posb) pos0 = posb[0];
    const long pos = (long)pos0 + (long)tt;
    const int lane = slot_of(threadIdx.x & 63), sub = lane & 7;
    if (pos < 0 || pos >= rows) {
        if ((threadIdx.x & 63) == 0) atomicOr(err, 1);
        return;
    }
    const int nb = M / 32;
    uint8_t * dst = cache + (size_t)pos * ((size_t)2 * nb * 34);
    f32x4 xv[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int b = it * 8 + (lane >> 3);
        const int bb = b < 2 * nb ? b : 0;
        const float * x = (bb < nb ? k + (size_t)tt * ldk : v + (size_t)tt * ldv) + (size_t)(bb % nb) * 32 + 4 * sub;
        xv[it] = __builtin_nontemporal_load((const f32x4 *)x);
    }
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int b = it * 8 + (lane >> 3);
        const bool active = b < 2 * nb;
        kv_q8_emit(xv[it], dst + (size_t)(active ? b : 0) * 34, sub, err, active);
    }
}

// pf_kv_append (q8_0 rows): no refusal rules; d stored as half, codes roundf(x * (1 / d)); err bit 1 for a row outside
__global__ void __launch_bounds__(256) pf_kv_append_rows(const float * __restrict__ k, int ldk, const float * __restrict__ v, int ldv, int M,
                                                         uint8_t * __restrict__ cache, int pos0, int rows, int * __restrict__ err,
                                                         const int32_t * __restrict__ posb = nullptr) {
    if (posb) pos0 = posb[0];
    const int tt = blockIdx.x; const long pos = (long)pos0 + tt;
    if (pos < 0 || pos >= rows) { if (threadIdx.x == 0) atomicOr(err, 1); return; }
    const int nb = M / 32, lane = slot_of(threadIdx.x & 63), sub = lane & 7;
    uint8_t * base = cache + (size_t)pos * ((size_t)2 * nb * 34);
    for (int b0 = (threadIdx.x >> 6) * 8; b0 < 2 * nb; b0 += 32) {
        const int b = b0 + (lane >> 3);
        const bool active = b < 2 * nb;
        const int bb = active ? b : 0;
        const float * x = (bb < nb ? k + (size_t)tt * ldk : v + (size_t)tt * ldv) + (size_t)(bb % nb) * 32 + 4 * sub;
        pf_q8_0_emit(*(const f32x4_a4 *)x, base + (size_t)bb * 34, sub, active);
    }
}
// a chunk of rows of at most 32 blocks (M <= 512, 16-byte aligned): a wave per row, as kv_q8_append_wave_rows
__global__ void __launch_bounds__(256) pf_kv_append_wave_rows(const float * __restrict__ k, int ldk, const float * __restrict__ v, int ldv, int M,
                                                              uint8_t * __restrict__ cache, int pos0, int rows, int T, int * __restrict__ err,
                                                              const int32_t * __restrict__ posb = nullptr) {
    const int tt = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tt >= T) return;
    if (posb) pos0 = posb[0];
    const long pos = (long)pos0 + tt;
    const int lane = slot_of(threadIdx.x & 63), sub = lane & 7;
    if (pos < 0 || pos >= rows) { if ((threadIdx.x & 63) == 0) atomicOr(err, 1); return; }
    const int nb = M / 32;
    uint8_t * dst = cache + (size_t)pos * ((size_t)2 * nb * 34);
    f32x4 xv[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int b = it * 8 + (lane >> 3);
        const int bb = b < 2 * nb ? b : 0;
        const float * x = (bb < nb ? k + (size_t)tt * ldk : v + (size_t)tt * ldv) + (size_t)(bb % nb) * 32 + 4 * sub;
        xv[it] = __builtin_nontemporal_load((const f32x4 *)x);
    }
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int b = it * 8 + (lane >> 3);
        const bool active = b < 2 * nb;
        pf_q8_0_emit(xv[it], dst + (size_t)(active ? b : 0) * 34, sub, active);
    }
}

// The reader: cache rows back to K / V values, value = (float)code * (float)half scale (one fp32 multiply, exact in the
// sense of the attention kernels' own decode: q3p_q8_stage, kernels/q3m_prefill.hip:617-632; host reference decode_q8_kv,
// python/caminus/ref_kv.py:127-144); F16: rounded to fp16 (the prefill staging's operand format). One workgroup per row,
// 8 lanes x 4 codes per block as in the writer; outputs leave as 16-byte (fp32) or 8-byte (fp16) stores per lane.
template <bool F16>
__global__ void __launch_bounds__(256) kv_q8_read_rows(const uint8_t * __restrict__ cache, const int32_t * __restrict__ row_ids, int pos0, int rows, int M,
                                                       void * __restrict__ k, int ldk, void * __restrict__ v, int ldv, int * __restrict__ err) {
    if (M < 32 || M % 32 || ldk < M || ldv < M || rows < 1) {
        if (threadIdx.x == 0) atomicOr(err, 4);
        return;
    }
    const size_t tt = blockIdx.x;
    const long pos = row_ids ? (long)row_ids[tt] : (long)pos0 + (long)blockIdx.x;
    if (pos < 0 || pos >= rows) {
        if (threadIdx.x == 0) atomicOr(err, 1);
        return;
    }
    const int nb = M / 32, lane = threadIdx.x & 63, sub = lane & 7;
    const uint8_t * src = cache + (size_t)pos * ((size_t)2 * nb * 34);
    for (int b0 = (threadIdx.x >> 6) * 8; b0 < 2 * nb; b0 += 32) {
        const int b = b0 + (lane >> 3);
        if (b >= 2 * nb) continue;
        const uint8_t * blk = src + (size_t)b * 34;
        const float d = h2f_bits(*(const uint16_t *)blk);
        const uint16_t * c = (const uint16_t *)(blk + 2 + 4 * sub);
        const uint32_t w = (uint32_t)c[0] | ((uint32_t)c[1] << 16);
        f32x4 y;
        y.x = (float)(int8_t)(w & 0xff) * d; y.y = (float)(int8_t)((w >> 8) & 0xff) * d;
        y.z = (float)(int8_t)((w >> 16) & 0xff) * d; y.w = (float)(int8_t)(w >> 24) * d;
        const size_t o = (b < nb ? tt * ldk : tt * ldv) + (size_t)(b % nb) * 32 + 4 * sub;
        if (F16) *(u32x2 *)((uint16_t *)(b < nb ? k : v) + o) = pack_f16x4(y);
        else *(f32x4_a4 *)((float *)(b < nb ? k : v) + o) = y;
    }
}

// The same reader for a chunk of rows with at most 32 blocks per row (M <= 512; row bytes a multiple of 16, 16-byte aligned cache): a
// wave per row, four rows per workgroup; the row comes in as 16-byte pieces straight to the wave's LDS (two requests per wave instead
// of three 2-byte loads per lane and block) and is decoded from there.
template <bool F16>
__global__ void __launch_bounds__(256) kv_q8_read_wave_rows(const uint8_t * __restrict__ cache, const int32_t * __restrict__ row_ids, int pos0, int rows, int M,
                                                            void * __restrict__ k, int ldk, void * __restrict__ v, int ldv, int T, int * __restrict__ err) {
    __shared__ __attribute__((aligned(16))) uint8_t stage_all[4][2 * 16 * 34];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, sub = lane & 7;
    const int tt = blockIdx.x * 4 + wave;
    if (tt >= T) return;
    const long pos = row_ids ? (long)row_ids[tt] : (long)pos0 + (long)tt;
    if (pos < 0 || pos >= rows) {
        if (lane == 0) atomicOr(err, 1);
        return;
    }
    const int nb = M / 32, rb = 2 * nb * 34, n16 = rb / 16;
    const uint8_t * src = cache + (size_t)pos * rb;
    uint8_t * stage = stage_all[wave];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int p = 64 * i + lane;
        const uint8_t * q = src + 16 * (size_t)p;
        if (p < n16)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)q, (__attribute__((address_space(3))) void *)(stage + 1024 * i), 16, 0, 2);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);                                    // vmcnt(0): the wave's own row has landed
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int b = it * 8 + (lane >> 3);
        if (b >= 2 * nb) continue;
        const uint8_t * blk = stage + (size_t)b * 34;
        const float d = h2f_bits(*(const uint16_t *)blk);
        const uint16_t * c = (const uint16_t *)(blk + 2 + 4 * sub);
        const uint32_t w = (uint32_t)c[0] | ((uint32_t)c[1] << 16);
        f32x4 y;
        y.x = (float)(int8_t)(w & 0xff) * d; y.y = (float)(int8_t)((w >> 8) & 0xff) * d;
        y.z = (float)(int8_t)((w >> 16) & 0xff) * d; y.w = (float)(int8_t)(w >> 24) * d;
        const size_t o = (b < nb ? (size_t)tt * ldk : (size_t)tt * ldv) + (size_t)(b % nb) * 32 + 4 * sub;
        if (F16) __builtin_nontemporal_store(pack_f16x4(y), (u32x2 *)((uint16_t *)(b < nb ? k : v) + o));
        else __builtin_nontemporal_store(y, (f32x4 *)((float *)(b < nb ? k : v) + o));
    }
}

// in-place orthonormal WHT of C chunks of n values, n in {64, 128, 256}: n / 4 lanes per chunk
template <int N>
__global__ void __launch_bounds__(256) hadamard_chunks(float * __restrict__ x, long C) {
    constexpr int LPC = N / 4;                       // lanes per chunk
    if (N == 128) {                                  // the 128-point transform with its lane stages on the DPP path (same pairs, same order)
        const int lane = slot_of(threadIdx.x & 63), l = lane & 31;
        const long c = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (c < C) v = __builtin_nontemporal_load((const f32x4 *)(x + c * 128 + 4 * l));
        v = hadamard128_l4(v, l, false);
        const float scale = 1.0f / sqrtf(128.0f);
        v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
        if (c < C) __builtin_nontemporal_store(v, (f32x4 *)(x + c * 128 + 4 * l));
        return;
    }
    const int lane = threadIdx.x & 63;
    const long wave = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long c = wave * (64 / LPC) + lane / LPC;
    const int l = lane % LPC;
    const bool active = c < C;
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (active) v = __builtin_nontemporal_load((const f32x4 *)(x + c * N + 4 * l));
    float a, b;
    a = v.x; b = v.y; v.x = a + b; v.y = a - b;
    a = v.z; b = v.w; v.z = a + b; v.w = a - b;
    a = v.x; b = v.z; v.x = a + b; v.z = a - b;
    a = v.y; b = v.w; v.y = a + b; v.w = a - b;
#pragma unroll
    for (int m = 1; m < LPC; m <<= 1) {
        const bool hi = (l & m) != 0;
        const float p0 = __shfl_xor(v.x, m, 64), p1 = __shfl_xor(v.y, m, 64), p2 = __shfl_xor(v.z, m, 64), p3 = __shfl_xor(v.w, m, 64);
        v.x = hi ? p0 - v.x : v.x + p0; v.y = hi ? p1 - v.y : v.y + p1;
        v.z = hi ? p2 - v.z : v.z + p2; v.w = hi ? p3 - v.w : v.w + p3;
    }
    const float scale = 1.0f / sqrtf((float)N);
    v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
    if (active) __builtin_nontemporal_store(v, (f32x4 *)(x + c * N + 4 * l));        // (in place and streamed: non-temporal both ways, 107 -> 94 us for 600 MB)
}

// OP_HADAMARD on the attention output followed by OP_GATE_MUL16 (python/caminus/engine/q35_dense.py:419-420: the dense Q8 line rotates the
// attention output back in chunks of 64 and multiplies it by the sigmoid of the gate half of the q projection): hadamard_chunks' transform
// (same pairs, same order, same scale) and gate_mul's fp32 -> fp16 form on the values as the first kernel would have stored them, in one
// pass; xo (optional) receives the transformed values, as the in-place op would leave them.
CAMX_DEV float kv_sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }      // gate_mul's form for 16-bit outputs
template <int N>
__global__ void __launch_bounds__(256) hadamard_gate16_k(const float * __restrict__ x, float * __restrict__ xo, const float * __restrict__ gate,
                                                         uint16_t * __restrict__ y16, long C, int D, int stride, int off) {
    constexpr int LPC = N / 4;
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    long c; int l; bool active;
    if (N == 128) {
        const int lane = slot_of(threadIdx.x & 63); l = lane & 31;
        c = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
        active = c < C;
        if (active) v = __builtin_nontemporal_load((const f32x4 *)(x + c * 128 + 4 * l));
        v = hadamard128_l4(v, l, false);
    } else {
        const int lane = threadIdx.x & 63;
        c = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPC) + lane / LPC;
        l = lane % LPC;
        active = c < C;
        if (active) v = __builtin_nontemporal_load((const f32x4 *)(x + c * N + 4 * l));
        float a, b;
        a = v.x; b = v.y; v.x = a + b; v.y = a - b;
        a = v.z; b = v.w; v.z = a + b; v.w = a - b;
        a = v.x; b = v.z; v.x = a + b; v.z = a - b;
        a = v.y; b = v.w; v.y = a + b; v.w = a - b;
#pragma unroll
        for (int m = 1; m < LPC; m <<= 1) {
            const bool hi = (l & m) != 0;
            const float p0 = __shfl_xor(v.x, m, 64), p1 = __shfl_xor(v.y, m, 64), p2 = __shfl_xor(v.z, m, 64), p3 = __shfl_xor(v.w, m, 64);
            v.x = hi ? p0 - v.x : v.x + p0; v.y = hi ? p1 - v.y : v.y + p1;
            v.z = hi ? p2 - v.z : v.z + p2; v.w = hi ? p3 - v.w : v.w + p3;
        }
    }
    const float scale = 1.0f / sqrtf((float)N);
    v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
    if (!active) return;
    const long e = c * N + 4 * l, h = e / D;
    const int d = (int)(e - h * D);
    if (xo) __builtin_nontemporal_store(v, (f32x4 *)(xo + e));
    const f32x4 g = __builtin_nontemporal_load((const f32x4 *)(gate + (size_t)h * stride + off + d));
    f32x4 o;
    o.x = v.x * kv_sigmoid_fast(g.x); o.y = v.y * kv_sigmoid_fast(g.y); o.z = v.z * kv_sigmoid_fast(g.z); o.w = v.w * kv_sigmoid_fast(g.w);
    __builtin_nontemporal_store(pack_f16x4(o), (u32x2 *)(y16 + e));
}

// out-of-place 128-point transform with the literal scale 0x1.6a09e6p-4f (the Q8 KV cache's rotation)
__global__ void __launch_bounds__(256) hadamard128_heads(const float * __restrict__ x, float * __restrict__ y, long heads) {
    const int lane = slot_of(threadIdx.x & 63);
    const long h = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
    const int l = lane & 31;
    const bool active = h < heads;
    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (active) v = x == y ? *(const f32x4 *)(x + h * 128 + 4 * l) : __builtin_nontemporal_load((const f32x4 *)(x + h * 128 + 4 * l));
    v = hadamard128_l4(v, l, true);
    if (active) __builtin_nontemporal_store(v, (f32x4 *)(y + h * 128 + 4 * l));
}

extern "C" {

static int own_kv_q8_append_launch(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, const int32_t * posb, int rows,
                                   int * err, int T, hipStream_t st) {
    if (!k || !v || !cache || !err || T < 0 || ((uintptr_t)k & 3) || ((uintptr_t)v & 3) || ((uintptr_t)cache & 1)) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const bool chunk = T >= 1024 && M >= 32 && M % 32 == 0 && M <= 512 && ldk >= M && ldv >= M && rows >= 1 &&
                       ((ldk | ldv) & 3) == 0 && (((uintptr_t)k | (uintptr_t)v) & 15) == 0;
    if (chunk) kv_q8_append_wave_rows<<<dim3((T + 3) / 4), dim3(256), 0, st>>>(k, ldk, v, ldv, M, cache, pos0, rows, T, err, posb);
    else kv_q8_append_rows<<<dim3(T), dim3(256), 0, st>>>(k, ldk, v, ldv, M, cache, pos0, rows, err, posb);
    CAMX_LAUNCH_RET();
}
int camx_own_kv_q8_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, int rows, int * err,
                          int T, hipStream_t st) {
    return own_kv_q8_append_launch(k, ldk, v, ldv, M, cache, pos0, nullptr, rows, err, T, st);
}

// The Q8 KV reader (no kernel of its own in the reference: the decode is inlined in its attention kernels). Row t = row_ids ?
// row_ids[t] : pos0 + t; k, v [T][ld] fp32 (f16 = 0) or fp16 bits (f16 = 1). err bits: 1 a row outside [0, rows) (its outputs
// stay untouched), 4 layout.
int camx_own_kv_q8_read(const uint8_t * cache, const int32_t * row_ids, int pos0, int rows, int M, void * k, int ldk, void * v, int ldv,
                        int * err, int T, int f16, hipStream_t st) {
    if (!cache || !k || !v || !err || T < 0 || ((uintptr_t)cache & 1) || ((uintptr_t)k & (f16 ? 7 : 3)) || ((uintptr_t)v & (f16 ? 7 : 3)) ||
        (f16 && ((ldk | ldv) & 3))) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    const bool chunk = T >= 1024 && M >= 32 && M % 32 == 0 && M <= 512 && (2 * (M / 32) * 34) % 16 == 0 && ldk >= M && ldv >= M && rows >= 1 &&
                       ((uintptr_t)cache & 15) == 0 && (f16 || ((((uintptr_t)k | (uintptr_t)v) & 15) == 0 && ((ldk | ldv) & 3) == 0));
    if (chunk) {
        if (f16) kv_q8_read_wave_rows<true><<<dim3((T + 3) / 4), dim3(256), 0, st>>>(cache, row_ids, pos0, rows, M, k, ldk, v, ldv, T, err);
        else kv_q8_read_wave_rows<false><<<dim3((T + 3) / 4), dim3(256), 0, st>>>(cache, row_ids, pos0, rows, M, k, ldk, v, ldv, T, err);
    }
    else if (f16) kv_q8_read_rows<true><<<dim3(T), dim3(256), 0, st>>>(cache, row_ids, pos0, rows, M, k, ldk, v, ldv, err);
    else kv_q8_read_rows<false><<<dim3(T), dim3(256), 0, st>>>(cache, row_ids, pos0, rows, M, k, ldk, v, ldv, err);
    CAMX_LAUNCH_RET();
}
static int pf_kv_append_launch(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, const int32_t * posb, int rows, int * err,
                               int T, hipStream_t st) {
    if (!k || !v || !cache || !err || T < 0 || M < 32 || M % 32 || ldk < M || ldv < M || ((uintptr_t)cache & 1)) return CAMX_EINVAL;
    if (T == 0) return CAMX_OK;
    if (T >= 1024 && M <= 512 && !(((uintptr_t)k | (uintptr_t)v) & 15) && !((ldk | ldv) & 3))
        pf_kv_append_wave_rows<<<dim3((T + 3) / 4), dim3(256), 0, st>>>(k, ldk, v, ldv, M, cache, pos0, rows, T, err, posb);
    else pf_kv_append_rows<<<dim3(T), dim3(256), 0, st>>>(k, ldk, v, ldv, M, cache, pos0, rows, err, posb);
    CAMX_LAUNCH_RET();
}
// (for camx_qk_nr_kv's prefill-sized batches, rope.hip: the same launcher with the position from a host integer or a device word)
int camx_i_pf_kv_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, const int32_t * posb, int rows, int * err,
                        int T, hipStream_t st) {
    return pf_kv_append_launch(k, ldk, v, ldv, M, cache, pos0, posb, rows, err, T, st);
}
int camx_pf_kv_append(const float * k, int ldk, const float * v, int ldv, int M, uint8_t * cache, int pos0, int rows, int * err,
                      int T, hipStream_t st) {
    return pf_kv_append_launch(k, ldk, v, ldv, M, cache, pos0, nullptr, rows, err, T, st);
}
// OP_KV_APPEND by its Seg fields (python/caminus/engine/k3.py:1065-1089; kernels/k3_gguf_ops.h:1520-1553, kernels/k3_q35_kvq8_ops.h:16-27): a = k,
// W = v (fp32 [T][M]), y = cache, asum = pos (int32 [1] on the device: token t goes to row pos[0] + t), N = M, gs = err. work 0: fp16 rows
// [K | V]; 1: ggml q8_0 rows (no refusal rules); 2: the dense Q8 line's blocks with the codec's refusal rules (the reference selects it by its
// K3_Q35_KV_Q8 build, with work = 1 and the error word in gs). rows = the cache's rows, checked on the device as the reference's launch guard
// does (err bit 1, the row is not written); err bit 2 a refused block, 4 layout (work 2).
int camx_i_kv_append16(const float * k, int ldk, const float * v, int ldv, uint16_t * cache, int M, int pos0, const int32_t * posb, int rows, int * err, int T, hipStream_t st);
int camx_op_kv_append(const float * k, const float * v, void * cache, const int32_t * pos, int M, int work, int * err, int rows, int T, hipStream_t st) {
    if (!pos || work < 0 || work > 2) return CAMX_EINVAL;
    if (work == 0) return camx_i_kv_append16(k, M, v, M, (uint16_t *)cache, M, 0, pos, rows, err, T, st);
    if (work == 1) return pf_kv_append_launch(k, M, v, M, M, (uint8_t *)cache, 0, pos, rows, err, T, st);
    return own_kv_q8_append_launch(k, M, v, M, M, (uint8_t *)cache, 0, pos, rows, err, T, st);
}
// OP_HADAMARD by its Seg fields (python/caminus/engine/k3.py:1244-1257): y = x (in place), N = C chunks, K = n, rows_per_task = chunks per task
int camx_pf_hadamard(float * x, int C, int n, int rpb, hipStream_t st);
int camx_op_hadamard(float * x, int C, int n, int rows_per_task, hipStream_t st) { return camx_pf_hadamard(x, C, n, rows_per_task, st); }

int camx_pf_hadamard(float * x, int C, int n, int rpb, hipStream_t st) {
    (void)rpb;
    if (!x || C < 0 || (n != 64 && n != 128 && n != 256) || ((uintptr_t)x & 15)) return CAMX_EINVAL;
    if (C == 0) return CAMX_OK;
    const int cpw = 256 / n;                                           // chunks per wave
    const unsigned blocks = (unsigned)(((long)C + 4 * cpw - 1) / (4 * cpw));
    if (n == 64) hadamard_chunks<64><<<dim3(blocks), dim3(256), 0, st>>>(x, C);
    else if (n == 128) hadamard_chunks<128><<<dim3(blocks), dim3(256), 0, st>>>(x, C);
    else hadamard_chunks<256><<<dim3(blocks), dim3(256), 0, st>>>(x, C);
    CAMX_LAUNCH_RET();
}

// OP_HADAMARD (chunks of hn values of a) then OP_GATE_MUL16 in one launch: a fp32 [n] (n = heads * dim values, dim % hn == 0), gate at
// (i / dim) * head_stride + offset + i % dim, out16 fp16 [n]; a_out (optional, may be a) = the transformed values. Equal to camx_op_hadamard
// followed by camx_op_gate_mul16 bit for bit.
int camx_op_hadamard_gate_mul16(const float * a, float * a_out, const float * gate, int head_stride, int offset, uint16_t * out16, int n, int dim, int hn,
                                hipStream_t st) {
    if (!a || !gate || !out16 || n < 0 || dim < 1 || (hn != 64 && hn != 128 && hn != 256) || dim % hn || n % dim || head_stride < dim || offset < 0 ||
        ((head_stride | offset) & 3) || (((uintptr_t)a | (uintptr_t)a_out | (uintptr_t)gate) & 15) || ((uintptr_t)out16 & 7)) return CAMX_EINVAL;
    if (n == 0) return CAMX_OK;
    const long C = n / hn;
    const int cpw = 256 / hn;
    const unsigned blocks = (unsigned)((C + 4 * cpw - 1) / (4 * cpw));
    if (hn == 64) hadamard_gate16_k<64><<<dim3(blocks), dim3(256), 0, st>>>(a, a_out, gate, out16, C, dim, head_stride, offset);
    else if (hn == 128) hadamard_gate16_k<128><<<dim3(blocks), dim3(256), 0, st>>>(a, a_out, gate, out16, C, dim, head_stride, offset);
    else hadamard_gate16_k<256><<<dim3(blocks), dim3(256), 0, st>>>(a, a_out, gate, out16, C, dim, head_stride, offset);
    CAMX_LAUNCH_RET();
}

int camx_hadamard128(const float * x, float * y, long heads, hipStream_t st) {
    if (!x || !y || heads < 0 || ((uintptr_t)x & 15) || ((uintptr_t)y & 15)) return CAMX_EINVAL;
    if (heads == 0) return CAMX_OK;
    hadamard128_heads<<<dim3((unsigned)((heads + 7) / 8)), dim3(256), 0, st>>>(x, y, heads);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
