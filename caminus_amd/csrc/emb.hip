// Quantized embedding-row gather + dequant for gfx950: GGUF Q4_K (144 B / 256 values) and Q8_0 (34 B / 32 values) rows to
// fp32 and / or bf16, optionally followed in the same wave by residual add + RMSNorm + q8_1 so the gathered row never
// returns to HBM. Replaces q3p_emb / OP_OWN_EMB (kernels/q3m_prefill.hip:364-380, kernels/k3_own_ops.h:279-304); the Q8_0
// arithmetic is the host decoder's (python/caminus/own_dequant.py:202-206).
//
// One wave per token row; slab j of 256 values = one Q4_K block or eight Q8_0 blocks; lane p decodes values 4p .. 4p + 3
// of each slab: for Q4_K one dword of nibbles per lane (lanes 8 apart share it: low / high nibble) and the 16-byte block
// header. y = (d * sc) * q - dmin * m with every product and the difference rounded separately.
#include "common.cuh"

enum { FMT_Q4_K = 0, FMT_Q8_0 = 1 };

CAMX_DEV f32x4 q4k_decode4(const uint8_t * blk, int lane) {
    const u32x4 hdr = *(const u32x4 *)blk;                       // d | dmin, then the 12 scale bytes
    const int sb = lane >> 3, is = sb >> 1, hi = sb & 1;
    const uint64_t s03 = (uint64_t)hdr.y, s47 = (uint64_t)hdr.z, s8b = (uint64_t)hdr.w;
    uint32_t sc, m;
    if (sb < 4) {
        sc = (uint32_t)(s03 >> (8 * sb)) & 63u;
        m = (uint32_t)(s47 >> (8 * sb)) & 63u;
    } else {
        const uint32_t hi8 = (uint32_t)(s8b >> (8 * (sb - 4))) & 0xffu;
        sc = (hi8 & 0xfu) | ((((uint32_t)(s03 >> (8 * (sb - 4))) & 0xffu) >> 6) << 4);
        m = (hi8 >> 4) | ((((uint32_t)(s47 >> (8 * (sb - 4))) & 0xffu) >> 6) << 4);
    }
    const float d = h2f_bits((uint16_t)(hdr.x & 0xffffu)), dm = h2f_bits((uint16_t)(hdr.x >> 16));
    const uint32_t qw = *(const uint32_t *)(blk + 16 + is * 32 + 4 * (lane & 7)) >> (4 * hi);
    const float dl = d * (float)sc, ml = dm * (float)m;
    f32x4 y;
    y.x = dl * (float)(qw & 15u) - ml; y.y = dl * (float)((qw >> 8) & 15u) - ml;
    y.z = dl * (float)((qw >> 16) & 15u) - ml; y.w = dl * (float)((qw >> 24) & 15u) - ml;
    return y;
}

CAMX_DEV f32x4 q80_decode4(const uint8_t * slab, int lane) {     // slab: 8 blocks of 34 bytes, 2-byte aligned
    const uint8_t * blk = slab + 34 * (lane >> 3);
    const float d = h2f_bits(*(const uint16_t *)blk);
    const uint16_t * c = (const uint16_t *)(blk + 2 + 4 * (lane & 7));
    const uint32_t w = (uint32_t)c[0] | ((uint32_t)c[1] << 16);
    f32x4 y;
    y.x = d * (float)(int8_t)(w & 0xff); y.y = d * (float)(int8_t)((w >> 8) & 0xff);
    y.z = d * (float)(int8_t)((w >> 16) & 0xff); y.w = d * (float)(int8_t)(w >> 24);
    return y;
}

struct EmbArgs {
    const uint8_t * W; long rb; int vocab;
    const int32_t * toks;
    float * x;               // optional fp32 [n][N]
    uint16_t * xbf;          // optional bf16 [n][N] (f2bf)
    int N, n;
    // fused tail (nw != null): x <- row (+ d), h = rmsnorm(x) * nw, optional copies
    const float * d;         // optional addend fp32 [n][N]
    const float * nw; float eps;
    float * h; uint16_t * h16; uint8_t * q8;
};

// EXACT: the row has exactly NI_MAX slabs (straight-line loops: the loads are issued as one batch)
template <int FMT, int NI_MAX, bool TAIL, bool EXACT>
__global__ void __launch_bounds__(256) emb_rows(EmbArgs a) {
    const int lane = slot_of(threadIdx.x & 63);
    const int t = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (t >= a.n) return;
    int tok = a.toks[t]; tok = tok < 0 ? 0 : tok; tok = tok > a.vocab - 1 ? a.vocab - 1 : tok;
    const uint8_t * row = a.W + (size_t)tok * a.rb;
    const int N = EXACT ? NI_MAX * 256 : a.N, ni = EXACT ? NI_MAX : N >> 8;
    // short rows: the addend and gamma do not depend on the token id, so they are requested before the table row is decoded
    // (one memory round trip after the id instead of three)
    constexpr bool PRE = TAIL;
    f32x4 gpre[PRE ? NI_MAX : 1], dpre[PRE ? NI_MAX : 1];
    if (PRE) {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) {
                gpre[j] = *(const f32x4 *)(a.nw + 256 * j + 4 * lane);
                if (a.d) dpre[j] = *(const f32x4 *)(a.d + (size_t)t * N + 256 * j + 4 * lane);
            }
    }
    // every table load first, then the stores: a load written after a store that might alias it cannot be hoisted above it,
    // and the row would cost one memory round trip per slab
    f32x4 xv[NI_MAX];
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni) xv[j] = FMT == FMT_Q4_K ? q4k_decode4(row + (size_t)j * 144, lane) : q80_decode4(row + (size_t)j * 272, lane);
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni) {
            const size_t o = (size_t)t * N + 256 * j + 4 * lane;
            if (!TAIL || !a.d) { if (a.x) *(f32x4 *)(a.x + o) = xv[j]; }
            if (a.xbf) *(u32x2 *)(a.xbf + o) = pack_f2bf_x4(xv[j]);
        }
    if (!TAIL) return;
    if (a.d) {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) {
                const size_t o = (size_t)t * N + 256 * j + 4 * lane;
                xv[j] = xv[j] + (PRE ? dpre[j] : *(const f32x4 *)(a.d + o));
                if (a.x) *(f32x4 *)(a.x + o) = xv[j];
            }
    }
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni) {
            ss.x = __builtin_fmaf(xv[j].x, xv[j].x, ss.x); ss.y = __builtin_fmaf(xv[j].y, xv[j].y, ss.y);
            ss.z = __builtin_fmaf(xv[j].z, xv[j].z, ss.z); ss.w = __builtin_fmaf(xv[j].w, xv[j].w, ss.w);
        }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)N + a.eps);
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni) {
            const f32x4 g = PRE ? gpre[j] : *(const f32x4 *)(a.nw + 256 * j + 4 * lane);
            f32x4 v;
            v.x = (xv[j].x * scale) * g.x; v.y = (xv[j].y * scale) * g.y; v.z = (xv[j].z * scale) * g.z; v.w = (xv[j].w * scale) * g.w;
            const size_t o = (size_t)t * N + 256 * j + 4 * lane;
            if (a.h) *(f32x4 *)(a.h + o) = v;
            if (a.h16) *(u32x2 *)(a.h16 + o) = pack_f16x4(v);
            if (a.q8) q8_1_emit(v, a.q8 + ((size_t)t * (N >> 5) + 8 * j + (lane >> 3)) * 36, lane & 7);
        }
}

template <int FMT>
static int launch_emb(const EmbArgs & a, hipStream_t st) {
    if (a.n <= 0) return CAMX_OK;
    const dim3 grid((a.n + 3) / 4), block(256);
    const int ni = a.N >> 8;
    const bool tail = a.nw != nullptr;
#define CAMX_EMB(NI, EX) (tail ? emb_rows<FMT, NI, true, EX><<<grid, block, 0, st>>>(a) : emb_rows<FMT, NI, false, EX><<<grid, block, 0, st>>>(a))
    if (ni == 8) CAMX_EMB(8, true); else if (ni == 16) CAMX_EMB(16, true); else if (ni == 20) CAMX_EMB(20, true); else if (ni == 4) CAMX_EMB(4, true);
    else if (ni <= 8) CAMX_EMB(8, false); else if (ni <= 16) CAMX_EMB(16, false); else if (ni <= 24) CAMX_EMB(24, false); else CAMX_EMB(32, false);
#undef CAMX_EMB
    CAMX_LAUNCH_RET();
}

static int emb_check(const EmbArgs & a, int fmt) {
    if (!a.W || !a.toks || a.N < 256 || a.N % 256 || a.N > 8192 || a.n < 0 || a.vocab < 1) return CAMX_EINVAL;
    if (a.rb < (long)(fmt == FMT_Q4_K ? a.N / 256 * 144 : a.N / 32 * 34)) return CAMX_EINVAL;
    if (fmt == FMT_Q4_K ? (((uintptr_t)a.W & 15) || (a.rb & 15)) : (((uintptr_t)a.W & 1) || (a.rb & 1))) return CAMX_EINVAL;
    if (((uintptr_t)a.x & 15) || ((uintptr_t)a.xbf & 7) || ((uintptr_t)a.d & 15) || ((uintptr_t)a.nw & 15) || ((uintptr_t)a.h & 15) ||
        ((uintptr_t)a.h16 & 7) || ((uintptr_t)a.q8 & 3)) return CAMX_EINVAL;
    return CAMX_OK;
}

extern "C" {

// q3p_emb: x [n][N] fp32 = the Q4_K rows toks[i] (rb bytes per row), ids clamped to [0, vocab)
int camx_q3p_emb(const uint8_t * W, int rb, int vocab, const int32_t * toks, float * x, int N, int n, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, nullptr, N, n, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr};
    if (!x || emb_check(a, FMT_Q4_K)) return CAMX_EINVAL;
    return launch_emb<FMT_Q4_K>(a, st);
}

// gather + dequant with fp32 and / or bf16 outputs; fmt 0 = Q4_K, 1 = Q8_0
int camx_emb_gather(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n, int fmt, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, xbf, N, n, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr};
    if ((!x && !xbf) || (fmt != FMT_Q4_K && fmt != FMT_Q8_0) || emb_check(a, fmt)) return CAMX_EINVAL;
    return fmt == FMT_Q4_K ? launch_emb<FMT_Q4_K>(a, st) : launch_emb<FMT_Q8_0>(a, st);
}

// gather + dequant + (x += d) + RMSNorm * nw with h fp32 / fp16 / q8_1 copies, one pass per row (all outputs optional
// except that at least one is given); x receives the residual row (after the add)
int camx_emb_gather_add_rms(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, const float * d,
                            const float * nw, float eps, float * h, uint16_t * h16, void * q8, int N, int n, int fmt, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, xbf, N, n, d, nw, eps, h, h16, (uint8_t *)q8};
    if (!nw || (!x && !xbf && !h && !h16 && !q8) || (fmt != FMT_Q4_K && fmt != FMT_Q8_0) || emb_check(a, fmt)) return CAMX_EINVAL;
    return fmt == FMT_Q4_K ? launch_emb<FMT_Q4_K>(a, st) : launch_emb<FMT_Q8_0>(a, st);
}

}   // extern "C"
