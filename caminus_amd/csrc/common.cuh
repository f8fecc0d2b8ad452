// Shared device helpers for the gfx950 (CDNA4, wave64) row kernels.
//
// Row layout used by every kernel here ("L4"): a wave owns a row (or a 128/256-value head / block); lane p holds the four
// consecutive elements 256 j + 4 p + k (k = 0..3) of each 256-element slab j, so every global access is one 128-bit
// load per lane and a wave instruction covers 1 KiB of contiguous memory.
//
// The reference's reductions are stated for 256 logical threads in 32-lane groups (thread t owns elements t, t + 256, ..;
// xor butterfly 16, 8, 4, 2, 1 inside each group of 32; the 8 group sums added in order). In L4, logical thread
// t = 4 p + k, so a group of 32 logical threads is 8 consecutive slots x 4 registers, and the butterfly becomes
// slot xor 4, slot xor 2, slot xor 1, then register pairs (k, k ^ 2) and (k, k ^ 1): the same pairs in the same order,
// hence the same bits. The group sums are then read with v_readlane from lanes 0, 8, .., 56 and added in order.
//
// Slots and lanes: the position p above is a logical slot; slot u lives in lane slot_to_lane(u), which differs from u
// only inside each group of 8: slots 4..7 sit in lanes 7..4. With that placement every slot exchange the kernels need is
// one DPP modifier on the consuming VALU op (no LDS crossbar): slot ^ 1 and slot ^ 2 are quad permutes, slot ^ 4 is
// row_half_mirror (lane 7 - l), slot ^ 8 is row_ror:8. Only slot ^ 16 takes a ds_swizzle. Kernels compute addresses from
// slot_of(lane); a wave still touches the same contiguous bytes per instruction.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

#define CAMX_DEV __device__ __forceinline__

// lane -> the logical slot it holds (and back: the map is an involution)
CAMX_DEV int slot_of(int lane) { const int s = lane & 7; return (lane & ~7) | (s < 4 ? s : 11 - s); }

// ---- slot exchanges (every lane of the exchanging group must be active) ---------------------------------------------------
CAMX_DEV float lane_xor1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false)); }   // quad_perm [1,0,3,2]
CAMX_DEV float lane_xor2(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false)); }   // quad_perm [2,3,0,1]
CAMX_DEV float lane_xor4(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false)); }  // row_half_mirror
CAMX_DEV float lane_xor8(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false)); }  // row_ror:8
CAMX_DEV float lane_xor16(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401f)); }              // swizzle SWAP,16
CAMX_DEV float lane_read(float v, int lane) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane)); }

// ---- the 32-value butterfly in L4 (8 lanes x 4 registers): every lane of the 8 gets the group's sum / max ----------------
CAMX_DEV float group32_sum(f32x4 v) {
    float a0 = v.x, a1 = v.y, a2 = v.z, a3 = v.w;
    a0 += lane_xor4(a0); a1 += lane_xor4(a1); a2 += lane_xor4(a2); a3 += lane_xor4(a3);   // logical xor 16
    a0 += lane_xor2(a0); a1 += lane_xor2(a1); a2 += lane_xor2(a2); a3 += lane_xor2(a3);   // logical xor 8
    a0 += lane_xor1(a0); a1 += lane_xor1(a1); a2 += lane_xor1(a2); a3 += lane_xor1(a3);   // logical xor 4
    const float w0 = a0 + a2, w1 = a1 + a3;                                               // logical xor 2
    return w0 + w1;                                                                       // logical xor 1
}
CAMX_DEV float group8_max(float a) {   // max over the 8 lanes of a group (order-free)
    a = fmaxf(a, lane_xor4(a)); a = fmaxf(a, lane_xor2(a)); a = fmaxf(a, lane_xor1(a));
    return a;
}
CAMX_DEV float group8_sum(float a) {   // xor 4, 2, 1 butterfly over 8 lanes (the MMQ quantizer's 8-thread sum)
    a += lane_xor4(a); a += lane_xor2(a); a += lane_xor1(a);
    return a;
}
// max |v| as a chain of fmaxf that starts from 0: a NaN is skipped, and four NaNs give 0 (the reference's amax of a block of NaNs), not NaN
CAMX_DEV float absmax4(f32x4 v) { return fmaxf(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))), 0.0f); }

// the 8 group sums of a wave added in order from 0.0f (0 + p0 is p0 for the non-negative sums used here)
CAMX_DEV float wave_groups_in_order(float g) {
    float tot = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; q++) tot += lane_read(g, 8 * q);
    return tot;
}
// only the first ng groups (a 128-wide head: 4)
template <int NG> CAMX_DEV float half_groups_in_order(float g, int base_lane) {
    float tot = 0.0f;
#pragma unroll
    for (int q = 0; q < NG; q++) tot += __shfl(g, base_lane + 8 * q, 64);
    return tot;
}

CAMX_DEV float rsqrt_exact(float v) { return 1.0f / sqrtf(v); }   // correctly rounded sqrt then divide (the contract)

// ---- conversions -----------------------------------------------------------------------------------------------------------
CAMX_DEV float bf2f(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
CAMX_DEV uint16_t f2bf(float f) {          // round to nearest even; any NaN -> 0x7fc0
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
CAMX_DEV uint16_t to_bf16(float f) {       // the same rounding without the NaN case
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
CAMX_DEV float rbf(float f) { return bf2f(f2bf(f)); }
// fp32 -> fp16 of a value that is already rounded to fp32: the empty asm keeps the backend from folding the producing
// multiply / fma and the convert into one mixed-precision instruction (v_fma_mix*: one rounding where the contract has two)
CAMX_DEV uint16_t f2h_bits(float f) { asm volatile("" : "+v"(f)); return __builtin_bit_cast(uint16_t, (_Float16)f); }
CAMX_DEV float h2f_bits(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
// fp32 -> fp16 -> fp32 of a value that is already rounded to fp32: the opaque copy keeps the backend from folding the
// producing fma and the convert into one mixed-precision instruction (one rounding instead of two)
CAMX_DEV float f16r(float x) { asm volatile("" : "+v"(x)); return (float)(_Float16)x; }

// two fp32 -> packed bf16 by the hardware convert (round to nearest even, denormals kept); a NaN comes out quiet with its
// payload, which is neither of the two software conventions above, so callers route NaN through those
CAMX_DEV uint32_t hw_pk_bf16(float lo, float hi) {
    const f32x2 in = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, bf16x2));
}
CAMX_DEV bool any_nan4(f32x4 v) { return (v.x != v.x) | (v.y != v.y) | (v.z != v.z) | (v.w != v.w); }
CAMX_DEV u32x2 pack_bf16x4_rne(f32x4 v) {  // to_bf16 of four values, packed little-endian
    u32x2 r;
    if (__builtin_expect(any_nan4(v), 0)) {
        r.x = (uint32_t)to_bf16(v.x) | ((uint32_t)to_bf16(v.y) << 16);
        r.y = (uint32_t)to_bf16(v.z) | ((uint32_t)to_bf16(v.w) << 16);
    } else { r.x = hw_pk_bf16(v.x, v.y); r.y = hw_pk_bf16(v.z, v.w); }
    return r;
}
CAMX_DEV u32x2 pack_f2bf_x4(f32x4 v) {     // f2bf of four values (NaN -> 0x7fc0), packed little-endian
    u32x2 r;
    if (__builtin_expect(any_nan4(v), 0)) {
        r.x = (uint32_t)f2bf(v.x) | ((uint32_t)f2bf(v.y) << 16);
        r.y = (uint32_t)f2bf(v.z) | ((uint32_t)f2bf(v.w) << 16);
    } else { r.x = hw_pk_bf16(v.x, v.y); r.y = hw_pk_bf16(v.z, v.w); }
    return r;
}
CAMX_DEV u32x2 pack_f16x4(f32x4 v) {
    u32x2 r;
    r.x = (uint32_t)f2h_bits(v.x) | ((uint32_t)f2h_bits(v.y) << 16);
    r.y = (uint32_t)f2h_bits(v.z) | ((uint32_t)f2h_bits(v.w) << 16);
    return r;
}
// fp16 of the products t * g rounded once (no intermediate fp32 rounding): the mixed-precision fma with a -0 addend (which keeps the
// sign of a zero product), low then high half of one register
CAMX_DEV uint32_t mul_pack_f16x2_once(float t0, float g0, float t1, float g1) {
    uint32_t r = 0;
    const float nz = -0.0f;
    asm("v_fma_mixlo_f16 %0, %1, %2, %3" : "+v"(r) : "v"(t0), "v"(g0), "v"(nz));
    asm("v_fma_mixhi_f16 %0, %1, %2, %3" : "+v"(r) : "v"(t1), "v"(g1), "v"(nz));
    return r;
}
CAMX_DEV f32x4 unpack_bf16x4(u32x2 w) {
    f32x4 r;
    r.x = __builtin_bit_cast(float, w.x << 16); r.y = __builtin_bit_cast(float, w.x & 0xffff0000u);
    r.z = __builtin_bit_cast(float, w.y << 16); r.w = __builtin_bit_cast(float, w.y & 0xffff0000u);
    return r;
}

// roundf (half away from zero) of a value known to fit int8 after rounding, as a signed byte in the low 8 bits
// trunc(v + copysign(0.49999997f, v)) equals roundf(v) for every float with |v| <= 256 (checked exhaustively on a CPU)
CAMX_DEV uint32_t round_i8(float v) { return (uint32_t)(int)(v + __builtin_copysignf(0.49999997f, v)) & 0xffu; }
CAMX_DEV uint32_t pack_round_i8x4(f32x4 v) {
    return round_i8(v.x) | (round_i8(v.y) << 8) | (round_i8(v.z) << 16) | (round_i8(v.w) << 24);
}

// the four codes roundf(x / d) of a lane (d > 0 or the block is all zero and never gets here), packed. The IEEE quotient
// t = fl(x / d) is only needed to decide on which side of a half-integer it falls. p = x * rcp(d) is within 3.8e-5 of the
// exact quotient for |x / d| <= 127 (rcp: 1 ulp; one more rounding), t within 4e-6 of it, and half-integers are floats, so
// whenever p is farther than 2^-13 from every half-integer, roundf(t) = roundf(p). Lanes that hold a closer value (about
// one in a thousand), an infinity or a NaN, or whose d is too small for rcp, divide.
CAMX_DEV uint32_t q8_codes4(f32x4 v, float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    float p[4] = {v.x * r, v.y * r, v.z * r, v.w * r};
    int c[4];
    bool safe = true;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        c[k] = (int)(p[k] + __builtin_copysignf(0.49999997f, p[k]));
        safe &= fabsf(p[k] - (float)c[k]) <= 0.4998f;               // (exact difference; false for NaN and for an infinite p)
    }
    if (!safe) {
        p[0] = v.x / d; p[1] = v.y / d; p[2] = v.z / d; p[3] = v.w / d;
#pragma unroll
        for (int k = 0; k < 4; k++) c[k] = (int)(p[k] + __builtin_copysignf(0.49999997f, p[k]));
    }
    return ((uint32_t)c[0] & 0xffu) | (((uint32_t)c[1] & 0xffu) << 8) | (((uint32_t)c[2] & 0xffu) << 16) | ((uint32_t)c[3] << 24);
}

// ---- q8_1 (ggml 36-byte block) of 32 values held by 8 lanes x 4 registers; sub = lane & 7 -------------------------------
// d = amax / 127, q = amax == 0 ? 0 : roundf(x / d), header half2(d, sum) with the butterfly sum. blk: the block's base.
CAMX_DEV void q8_1_emit(f32x4 v, uint8_t * blk, int sub) {
    const float amax = group8_max(absmax4(v));
    const float sum = group32_sum(v);
    const float d = amax / 127.0f;
    uint32_t q = 0;
    if (amax != 0.0f) q = q8_codes4(v, d);
    *(uint32_t *)(blk + 4 + 4 * sub) = q;
    if (sub == 0) *(uint32_t *)blk = (uint32_t)f2h_bits(d) | ((uint32_t)f2h_bits(sum) << 16);
}

// ---- q8_0 (ggml 34-byte block) of 32 values held by 8 lanes x 4 registers; sub = lane & 7 -------------------------------
// d = amax / 127 stored as half, codes roundf(x * (1 / d)) (the cache writer's form: kernels/k3_gguf_ops.h:1520-1553). Every lane of
// the group takes part in the max; active = false: no store.
CAMX_DEV void pf_q8_0_emit(f32x4 xv, uint8_t * blk, int sub, bool active) {        // 8 lanes x 4 values: one block
    const float amax = group8_max(absmax4(xv));
    const float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    if (!active) return;
    f32x4 t; t.x = xv.x * id; t.y = xv.y * id; t.z = xv.z * id; t.w = xv.w * id;
    const uint32_t q = pack_round_i8x4(t);
    uint16_t * o = (uint16_t *)(blk + 2 + 4 * sub);
    o[0] = (uint16_t)q; o[1] = (uint16_t)(q >> 16);
    if (sub == 0) *(uint16_t *)blk = f2h_bits(d);
}

// ---- q8_1 block of 32 consecutive floats in LDS, all of it in one lane -------------------------------------------------------
// in: the block's 32 values; out: its 9 dwords (LDS); rot: the lane's number (the pieces are read in the order rot, rot + 1, ..
// mod 8, so that the lanes of a request fall on different banks). The sum keeps the 32-thread butterfly's tree (xor 16, 8, 4, 2, 1
// over one value per thread): its first three levels add the 4-value pieces c and c + 4, then c and c + 2, then the last two, its
// last two levels the four sums left; each level pairs pieces half a period apart, so the rotation changes no operand pair, and
// max and the codes do not depend on order. Codes: v * (1 / d) rounded to nearest is roundf(v / d) whenever it is farther than
// 2^-15 from a half-integer (|v / d| <= 127 and the refined reciprocal is within an ulp); a piece in which some lane's value is
// closer, infinite or NaN is redone with the division (every lane of the wave must be here: the decision is a ballot).
// MODE 1: the values are silu(v * rs) first (OP_GG_Q8_1's mode 1).
CAMX_DEV float silu_div(float x) { return x / (1.0f + expf(-x)); }
template <int MODE>
CAMX_DEV void q8_1_block_lane(const float * in, uint32_t * out, int rot, float rs, bool active = true) {   // active = false: every step but the stores
    f32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = *(const f32x4 *)(in + 4 * ((k + rot) & 7));
    if (MODE == 1) {
#pragma unroll
        for (int k = 0; k < 8; k++) { v[k].x = silu_div(v[k].x * rs); v[k].y = silu_div(v[k].y * rs); v[k].z = silu_div(v[k].z * rs); v[k].w = silu_div(v[k].w * rs); }
    }
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) amax = fmaxf(amax, absmax4(v[k]));
    const f32x4 s0 = v[0] + v[4], s1 = v[1] + v[5], s2 = v[2] + v[6], s3 = v[3] + v[7];
    const f32x4 u0 = s0 + s2, u1 = s1 + s3;
    const f32x4 w = u0 + u1;
    const float w0 = w.x + w.z, w1 = w.y + w.w;
    const float sum = w0 + w1;
    const float d = amax / 127.0f;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();       // (out may lie where other lanes' values were)
    if (active) out[0] = (uint32_t)f2h_bits(d) | ((uint32_t)f2h_bits(sum) << 16);
    float r = __builtin_amdgcn_rcpf(d);
    r = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
#pragma unroll
    for (int k = 0; k < 8; k++) {
        float p[4] = {v[k].x * r, v[k].y * r, v[k].z * r, v[k].w * r};
        int c[4];
        bool safe = true;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float n = __builtin_rintf(p[e]);
            safe &= fabsf(p[e] - n) <= 0.49996948f;                        // (false for NaN and for an infinite p)
            c[e] = (int)n;
        }
        if (__builtin_amdgcn_ballot_w64(!safe && amax != 0.0f) != 0) {
            p[0] = v[k].x / d; p[1] = v[k].y / d; p[2] = v[k].z / d; p[3] = v[k].w / d;
#pragma unroll
            for (int e = 0; e < 4; e++) c[e] = (int)(p[e] + __builtin_copysignf(0.49999997f, p[e]));
        }
        const uint32_t codes = ((uint32_t)c[0] & 0xffu) | (((uint32_t)c[1] & 0xffu) << 8) | (((uint32_t)c[2] & 0xffu) << 16) | ((uint32_t)c[3] << 24);
        if (active) out[1 + ((k + rot) & 7)] = amax != 0.0f ? codes : 0u;
    }
}
// The q8_1 blocks of a row that sits in this wave's LDS in element order (seg: nb32 * 32 floats, nb32 a multiple of 8): lane l quantizes
// block 64 p + l of pass p whole; the 9-dword blocks of a pass are staged over the values the pass has consumed and leave as 16-byte
// stores to dst (16-byte aligned; 36 nb32 bytes). Every lane of the wave calls it.
CAMX_DEV void q8_1_row_from_lds(float * seg, int nb32, uint8_t * dst, int lraw) {
    for (int p0 = 0; p0 < nb32; p0 += 64) {
        const int nbp = nb32 - p0 < 64 ? nb32 - p0 : 64;            // blocks of this pass
        float * in = seg + 32 * p0;
        uint32_t * stage = (uint32_t *)in;
        const bool on = lraw < nbp;
        q8_1_block_lane<0>(in + 32 * (on ? lraw : 0), stage + 9 * lraw, lraw, 0.0f, on);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
        u32x4 * d16 = (u32x4 *)(dst + (size_t)p0 * 36);
        const int n16 = nbp * 9 / 4;                                 // 16-byte pieces of the pass (nbp % 8 == 0)
        for (int i = lraw; i < n16; i += 64) __builtin_nontemporal_store(*(const u32x4 *)(stage + 4 * i), d16 + i);
    }
}

// ---- Q8 KV wire block (34 bytes) of 32 values held by 8 lanes x 4 registers ----------------------------------------------
// amax / 127, its fp32 reciprocal, roundf(x * inv), only the stored scale rounded to half. A refused block (non-finite
// input; nonzero block whose scale underflows, whose reciprocal overflows or whose half scale is not finite) keeps its
// bytes and ORs 2 into *err. blk is 2-byte aligned. Returns true when the block was written.
CAMX_DEV bool kv_q8_emit(f32x4 v, uint8_t * blk, int sub, int * err, bool active) {
    const bool fin = __builtin_isfinite(v.x) && __builtin_isfinite(v.y) && __builtin_isfinite(v.z) && __builtin_isfinite(v.w);
    const float amax = group8_max(fin ? absmax4(v) : INFINITY);
    const float d = amax / 127.0f;
    const float inv = d != 0.0f ? 1.0f / d : 0.0f;
    const _Float16 stored = (_Float16)d;
    const bool refuse = !__builtin_isfinite(amax) ||
                        (amax != 0.0f && (d == 0.0f || !__builtin_isfinite(d) || !__builtin_isfinite(inv) || !__builtin_isfinite((float)stored)));
    if (!active) return false;
    if (refuse) { if (sub == 0) atomicOr(err, 2); return false; }
    f32x4 t; t.x = v.x * inv; t.y = v.y * inv; t.z = v.z * inv; t.w = v.w * inv;
    const uint32_t q = pack_round_i8x4(t);
    uint16_t * o = (uint16_t *)(blk + 2 + 4 * sub);
    o[0] = (uint16_t)q; o[1] = (uint16_t)(q >> 16);
    if (sub == 0) *(uint16_t *)blk = __builtin_bit_cast(uint16_t, stored);
    return true;
}

// ---- the orthonormal 128-point Walsh-Hadamard transform of a head held by 32 lanes x 4 registers (element 4 l + k) ------
// stages h = 1, 2 pair registers, h = 4 .. 64 pair lanes l ^ 1 .. l ^ 16; pair (i, i + h) -> (a + b, a - b); then times
// 0x1.6a09e6p-4f. lane: the lane's index inside its 32-lane half.
CAMX_DEV f32x4 hadamard128_l4(f32x4 v, int lane, bool scale) {
    float a, b;
    a = v.x; b = v.y; v.x = a + b; v.y = a - b;
    a = v.z; b = v.w; v.z = a + b; v.w = a - b;
    a = v.x; b = v.z; v.x = a + b; v.z = a - b;
    a = v.y; b = v.w; v.y = a + b; v.w = a - b;
    // a cross-lane stage is (own + partner) in the lower lane and (partner - own) in the upper one: the upper lane's sign is
    // flipped first (exact), then both add the partner's value, which rides on the add as a DPP source where a row move does it.
    // (The elements are copied to scalars first: a bit cast applied straight to a vector element reads element 0.)
    float e[4] = {v.x, v.y, v.z, v.w};
#define CAMX_HSTAGE_DPP(BIT, CTRL)                                                                                  \
    {                                                                                                                 \
        const uint32_t m = (lane & BIT) ? 0x80000000u : 0u;                                                           \
        _Pragma("unroll") for (int k = 0; k < 4; k++) {                                                               \
            const float own = e[k];                                                                                   \
            const float p = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, own), CTRL, 0xf, 0xf, true));  \
            e[k] = p + __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, own) ^ m);                              \
        }                                                                                                             \
    }
    CAMX_HSTAGE_DPP(1, 0xB1) CAMX_HSTAGE_DPP(2, 0x4E) CAMX_HSTAGE_DPP(4, 0x141) CAMX_HSTAGE_DPP(8, 0x128)
#undef CAMX_HSTAGE_DPP
    {
        const uint32_t m = (lane & 16) ? 0x80000000u : 0u;
#pragma unroll
        for (int k = 0; k < 4; k++) { const float own = e[k]; e[k] = lane_xor16(own) + __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, own) ^ m); }
    }
    v.x = e[0]; v.y = e[1]; v.z = e[2]; v.w = e[3];
    if (scale) { v.x *= 0x1.6a09e6p-4f; v.y *= 0x1.6a09e6p-4f; v.z *= 0x1.6a09e6p-4f; v.w *= 0x1.6a09e6p-4f; }
    return v;
}

// ---- the small tables of a bf16 gate ---------------------------------------------------------------------------------------------
// 8192 entries cover +-0 and 2^-24 <= |g| < 2^8 (less two values): positive gates first, then negative ones; a kernel that looks
// gates up from LDS holds these and goes to the full 65536-entry table in device memory for a gate outside them.
#define SWS_A0 0x3380u                 // bf16 bits of 2^-24: the first magnitude
#define SWS_SPAN 0x0fffu               // magnitudes per sign; index SWS_SPAN is the entry of +-0 (and the stand-in of every gate outside the table)
#define SWS_TAB (2 * (SWS_SPAN + 1))
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
// the entries of two packed gates (16 bits each); outside: set when one of them is not in the table
CAMX_DEV uint32_t small_index2(uint32_t w, bool & outside) {
    const u16x2 a2 = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
    const u16x2 i2 = __builtin_elementwise_min(a2 - (u16x2){SWS_A0, SWS_A0}, (u16x2){SWS_SPAN, SWS_SPAN});      // below the table: wraps, clamps
    const u16x2 lo = a2 - (u16x2){1, 1};                                                                       // (a zero wraps to 0xffff: inside)
    outside |= (lo.x < SWS_A0 - 1) | (lo.y < SWS_A0 - 1) | (a2.x >= SWS_A0 + SWS_SPAN) | (a2.y >= SWS_A0 + SWS_SPAN);
    return ((w >> 3) & 0x10001000u) | __builtin_bit_cast(uint32_t, i2);                                        // the sign in bit 12
}

// ---- host-side helpers -------------------------------------------------------------------------------------------------------
#define CAMX_OK 0
#define CAMX_EINVAL 1     // hipErrorInvalidValue
#define CAMX_LAUNCH_RET() return (int)hipGetLastError()
