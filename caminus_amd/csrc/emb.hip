// Quantized embedding-row gather + dequant for gfx950: GGUF Q4_K (144 B / 256 values), Q8_0 (34 B / 32 values), IQ4_XS
// (136 B / 256) and IQ2_S (82 B / 256) rows to fp32 and / or bf16, optionally followed in the same wave by residual add +
// RMSNorm + q8_1 so the gathered row never returns to HBM; and the IQ4_NL rows (18 B / 32) of a per-layer-embedding feed.
// Replaces q3p_emb / OP_OWN_EMB (kernels/q3m_prefill.hip:364-380, kernels/k3_own_ops.h:279-304), embd_rows_iq4xs and
// ple_rows_iq4nl (kernels/prefill_feed.hip:24-54) and q35t_op_emb's IQ2_S rows (kernels/k3_q35t_ops.h:147-175); the Q8_0
// arithmetic is the host decoder's (python/caminus/own_dequant.py:202-206).
//
// One wave per token row; slab j of 256 values = one Q4_K block or eight Q8_0 blocks; lane p decodes values 4p .. 4p + 3
// of each slab: for Q4_K one dword of nibbles per lane (lanes 8 apart share it: low / high nibble) and the 16-byte block
// header. y = (d * sc) * q - dmin * m with every product and the difference rounded separately.
#include "common.cuh"
#include "iq2s_grid.inc"

enum { FMT_Q4_K = 0, FMT_Q8_0 = 1, FMT_IQ4_XS = 2, FMT_IQ2_S = 3, FMT_COUNT = 4 };
enum { ERR_PLE_INDEX = 1, ERR_TOKEN = 2 };

CAMX_DEV f32x4 q4k_decode4(const uint8_t * blk, int lane) {
    const u32x4 hdr = *(const u32x4 *)blk;                       // d | dmin, then the 12 scale bytes
    const int sb = lane >> 3, is = sb >> 1, hi = sb & 1;
    const uint32_t sh = 8 * (sb & 3);                                    // the sub-block's byte inside each scale word
    const uint32_t b03 = (hdr.y >> sh) & 0xffu, b47 = (hdr.z >> sh) & 0xffu, b8b = (hdr.w >> sh) & 0xffu;
    uint32_t sc, m;
    if (sb < 4) { sc = b03 & 63u; m = b47 & 63u; }
    else { sc = (b8b & 0xfu) | ((b03 >> 6) << 4); m = (b8b >> 4) | ((b47 >> 6) << 4); }
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

// the 16 values of IQ4_NL / IQ4_XS (-127 -104 -83 -65 -49 -35 -22 -10 1 13 25 38 53 69 89 113) for four 4-bit indices
// held one per byte: two byte permutes over the table's halves, then a select on bit 3
CAMX_DEV f32x4 iq4_values(uint32_t idx4) {
    const uint32_t sel = idx4 & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(0xf6eaddcfu, 0xbfad9881u, sel), hi = __builtin_amdgcn_perm(0x71594535u, 0x26190d01u, sel);
    const uint32_t top = ((idx4 >> 3) & 0x01010101u) * 0xffu;
    const uint32_t v = (hi & top) | (lo & ~top);
    f32x4 y;
    y.x = (float)(int8_t)(v & 0xff); y.y = (float)(int8_t)((v >> 8) & 0xff); y.z = (float)(int8_t)((v >> 16) & 0xff); y.w = (float)(int8_t)(v >> 24);
    return y;
}

// block_iq4_xs: f16 d, u16 scales_h, u8 scales_l[4], u8 qs[128]; sub-block ib (32 values): 6-bit scale ls, values
// qs[16 ib ..] low nibbles then high; y = (d * (ls - 32)) * value
CAMX_DEV f32x4 iq4xs_decode4(const uint8_t * blk, int lane) {
    const u32x2 hdr = *(const u32x2 *)blk;
    const int ib = lane >> 3;
    const uint32_t sh = hdr.x >> 16, sl = (hdr.y >> (8 * (ib >> 1))) & 0xffu;
    const int ls = (int)(((sl >> (4 * (ib & 1))) & 15u) | (((sh >> (2 * ib)) & 3u) << 4));
    const float dl = h2f_bits((uint16_t)(hdr.x & 0xffffu)) * (float)(ls - 32);
    const uint32_t qw = *(const uint32_t *)(blk + 8 + 16 * ib + 4 * (lane & 3)) >> (4 * ((lane >> 2) & 1));
    const f32x4 k = iq4_values(qw & 0x0f0f0f0fu);
    f32x4 y; y.x = dl * k.x; y.y = dl * k.y; y.z = dl * k.z; y.w = dl * k.w;
    return y;
}

// block_iq2_s: f16 d, qs[32] (low 8 bits of a 10-bit grid index per 8 values), signs[32] (a bit per value), qh[8] (the
// indices' high bits, four per byte), scales[8] (a nibble per 16 values); y = +-(((d * (0.5 + s)) * 0.25) * magnitude)
CAMX_DEV f32x4 iq2s_decode4(const uint8_t * blk, int lane) {
    const int ib = lane >> 3, g = (lane >> 1) & 3, h = lane & 1;
    const float d = h2f_bits(*(const uint16_t *)blk);
    const uint32_t idx = (uint32_t)blk[2 + 4 * ib + g] | ((((uint32_t)blk[66 + ib] >> (2 * g)) & 3u) << 8);
    const uint32_t m4 = IQ2S_MAG[2 * idx + h];
    const uint32_t sg = (uint32_t)blk[34 + 4 * ib + g] >> (4 * h);
    const float sc = (float)(((uint32_t)blk[74 + ib] >> (4 * ((lane >> 2) & 1))) & 15u);
    const float db = (d * (0.5f + sc)) * 0.25f;
    f32x4 y;
    y.x = db * (float)(m4 & 0xffu); y.y = db * (float)((m4 >> 8) & 0xffu); y.z = db * (float)((m4 >> 16) & 0xffu); y.w = db * (float)(m4 >> 24);
    if (sg & 1u) y.x = -y.x;
    if (sg & 2u) y.y = -y.y;
    if (sg & 4u) y.z = -y.z;
    if (sg & 8u) y.w = -y.w;
    return y;
}

template <int FMT> CAMX_DEV f32x4 emb_decode4(const uint8_t * row, int j, int lane) {
    if (FMT == FMT_Q4_K) return q4k_decode4(row + (size_t)j * 144, lane);
    if (FMT == FMT_Q8_0) return q80_decode4(row + (size_t)j * 272, lane);
    if (FMT == FMT_IQ4_XS) return iq4xs_decode4(row + (size_t)j * 136, lane);
    return iq2s_decode4(row + (size_t)j * 82, lane);
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
    int * err;               // optional: bit ERR_TOKEN is set when an id lies outside [0, vocab) (the id is clamped either way)
    int stream;              // set by the launcher for large batches: the gathered rows leave as non-temporal stores
    int key;                 // one token, given as the low half's complement of a 64-bit argmax key word at toks (OP_OWN_EMB's chained draft step)
};

// EXACT: the row has exactly NI_MAX slabs (straight-line loops: the loads are issued as one batch)
// SPLIT (batches too small to fill the chip): a workgroup per row. Every wave decodes the row and, with a tail, walks the same
// sum of squares (the same operations on the same values: the same bits in all four), but converts, quantizes and stores only
// the slabs j = wave (mod 4): the serial part behind the reduction, eight q8_1 slabs for a 2048-wide row, is a quarter as long.
// QL (wave-per-row batches with a q8_1 copy): the normed row goes to the wave's own LDS and lane l quantizes block l whole, instead of eight
// lanes sharing a block and each repeating its divide and two butterflies (105 instructions per lane and slab; the fused Q4_K row is bound by
// its instruction count: 1565 per wave)
template <int FMT, int NI_MAX, bool TAIL, bool EXACT, bool SPLIT = false, bool QL = false>
__global__ void __launch_bounds__(256) emb_rows(EmbArgs a) {
    __shared__ __attribute__((aligned(16))) float qrows[QL ? 4 : 1][QL ? NI_MAX * 256 : 4];
    const int lane = slot_of(threadIdx.x & 63), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = SPLIT ? blockIdx.x : blockIdx.x * 4 + wave;
    if (t >= a.n) return;
    auto mine = [&](int j) { return !SPLIT || (j & 3) == wave; };
    int tok = a.key ? (int)~(uint32_t)((const unsigned long long *)a.toks)[0] : a.toks[t];
    if (a.err && (tok < 0 || tok >= a.vocab) && lane == 0) atomicOr(a.err, ERR_TOKEN);
    tok = tok < 0 ? 0 : tok; tok = tok > a.vocab - 1 ? a.vocab - 1 : tok;
    const uint8_t * row = a.W + (size_t)tok * a.rb;
    const int N = EXACT ? NI_MAX * 256 : a.N, ni = EXACT ? NI_MAX : N >> 8;
    // short rows: the addend and gamma do not depend on the token id, so they are requested before the table row is decoded
    // (one memory round trip after the id instead of three)
    constexpr bool PRE = TAIL && SPLIT;      // (wave-per-row batches are bound by their waves per SIMD: 64 fewer registers without the early copies)
    f32x4 gpre[PRE ? NI_MAX : 1], dpre[PRE ? NI_MAX : 1];
    if (PRE) {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) {
                if (mine(j) && !(SPLIT && EXACT && NI_MAX % 4 == 0)) gpre[j] = *(const f32x4 *)(a.nw + 256 * j + 4 * lane);
                if (a.d) dpre[j] = *(const f32x4 *)(a.d + (size_t)t * N + 256 * j + 4 * lane);
            }
    }
    // every table load first, then the stores: a load written after a store that might alias it cannot be hoisted above it,
    // and the row would cost one memory round trip per slab
    f32x4 xv[NI_MAX];
    if (SPLIT && TAIL && FMT != FMT_Q8_0) {
        // a workgroup per row with a tail: each wave decodes its own slabs and the four share them through LDS (with one wave per SIMD
        // every instruction of a wave is latency: 270 fewer of them per wave than decoding a Q4_K row four times; Q8_0 decodes in two
        // loads and four converts per lane, which the exchange does not beat)
        __shared__ f32x4 xs[NI_MAX][64];
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && mine(j)) { xv[j] = emb_decode4<FMT>(row, j, lane); xs[j][lane] = xv[j]; }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && !mine(j)) xv[j] = xs[j][lane];
    } else {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && (TAIL || mine(j))) xv[j] = emb_decode4<FMT>(row, j, lane);
    }
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni && mine(j)) {
            const size_t o = (size_t)t * N + 256 * j + 4 * lane;
            if (!TAIL && a.stream) {
                if (a.x) __builtin_nontemporal_store(xv[j], (f32x4 *)(a.x + o));
                if (a.xbf) __builtin_nontemporal_store(pack_f2bf_x4(xv[j]), (u32x2 *)(a.xbf + o));
            } else {
                if (!TAIL || !a.d) { if (a.x) *(f32x4 *)(a.x + o) = xv[j]; }
                if (a.xbf) *(u32x2 *)(a.xbf + o) = pack_f2bf_x4(xv[j]);
            }
        }
    if (!TAIL) return;
    if (a.d) {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) {
                const size_t o = (size_t)t * N + 256 * j + 4 * lane;
                xv[j] = xv[j] + (PRE ? dpre[j] : *(const f32x4 *)(a.d + o));
                if (a.x && mine(j)) *(f32x4 *)(a.x + o) = xv[j];
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
    if (SPLIT && EXACT && NI_MAX % 4 == 0) {
        // the wave's slabs wave, wave + 4, .. picked out of the register array by selects on the (uniform) wave number, so that their
        // conversions and q8_1 blocks are one straight run of code and overlap each other's latencies
#pragma unroll
        for (int s = 0; s < NI_MAX / 4; s++) {
            const int j = wave + 4 * s;
            const f32x4 xa = wave == 0 ? xv[4 * s] : wave == 1 ? xv[4 * s + 1] : wave == 2 ? xv[4 * s + 2] : xv[4 * s + 3];
            const f32x4 g = *(const f32x4 *)(a.nw + 256 * j + 4 * lane);
            f32x4 v;
            v.x = (xa.x * scale) * g.x; v.y = (xa.y * scale) * g.y; v.z = (xa.z * scale) * g.z; v.w = (xa.w * scale) * g.w;
            const size_t o = (size_t)t * N + 256 * j + 4 * lane;
            if (a.h) *(f32x4 *)(a.h + o) = v;
            if (a.h16) *(u32x2 *)(a.h16 + o) = pack_f16x4(v);
            if (a.q8) q8_1_emit(v, a.q8 + ((size_t)t * (N >> 5) + 8 * j + (lane >> 3)) * 36, lane & 7);
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni && mine(j)) {
            const f32x4 g = PRE ? gpre[j] : *(const f32x4 *)(a.nw + 256 * j + 4 * lane);
            f32x4 v;
            v.x = (xv[j].x * scale) * g.x; v.y = (xv[j].y * scale) * g.y; v.z = (xv[j].z * scale) * g.z; v.w = (xv[j].w * scale) * g.w;
            const size_t o = (size_t)t * N + 256 * j + 4 * lane;
            if (a.h) *(f32x4 *)(a.h + o) = v;
            if (a.h16) *(u32x2 *)(a.h16 + o) = pack_f16x4(v);
            if (QL) *(f32x4 *)(qrows[wave] + 256 * j + 4 * lane) = v;
            else if (a.q8) q8_1_emit(v, a.q8 + ((size_t)t * (N >> 5) + 8 * j + (lane >> 3)) * 36, lane & 7);
        }
    if (QL) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();          // the wave's row is in LDS
        q8_1_row_from_lds(qrows[wave], N >> 5, a.q8 + (size_t)t * (N >> 5) * 36, threadIdx.x & 63);
    }
}

template <int FMT>
static int launch_emb(const EmbArgs & a0, hipStream_t st) {
    if (a0.n <= 0) return CAMX_OK;
    EmbArgs a = a0;
    a.stream = (long)a.n * a.N >= (1L << 20);
    const dim3 block(256);
    const int ni = a.N >> 8;
    const bool tail = a.nw != nullptr;
    // a workgroup per row while the chip is not full: 256 rows x 4 waves are one wave per SIMD; from 512 rows on the four-fold decode costs
    // more than the shorter tail saves (2048-wide Q4_K rows with the fused tail: 6.6 us at 256 rows, 12.0 at 512 against 8 before)
    if (a.n <= 256 && (ni == 4 || ni == 8 || ni == 16 || ni == 20)) {
        const dim3 grid(a.n);
#define CAMX_EMB_SPLIT(NI) (tail ? emb_rows<FMT, NI, true, true, true><<<grid, block, 0, st>>>(a) : emb_rows<FMT, NI, false, true, true><<<grid, block, 0, st>>>(a))
        if (ni == 8) CAMX_EMB_SPLIT(8); else if (ni == 16) CAMX_EMB_SPLIT(16); else if (ni == 20) CAMX_EMB_SPLIT(20); else CAMX_EMB_SPLIT(4);
#undef CAMX_EMB_SPLIT
        CAMX_LAUNCH_RET();
    }
    const dim3 grid((a.n + 3) / 4);
    if (tail && a.q8 && ((uintptr_t)a.q8 & 15) == 0 && (ni == 4 || ni == 8 || ni == 16)) {
        if (ni == 8) emb_rows<FMT, 8, true, true, false, true><<<grid, block, 0, st>>>(a);
        else if (ni == 16) emb_rows<FMT, 16, true, true, false, true><<<grid, block, 0, st>>>(a);
        else emb_rows<FMT, 4, true, true, false, true><<<grid, block, 0, st>>>(a);
        CAMX_LAUNCH_RET();
    }
#define CAMX_EMB(NI, EX) (tail ? emb_rows<FMT, NI, true, EX><<<grid, block, 0, st>>>(a) : emb_rows<FMT, NI, false, EX><<<grid, block, 0, st>>>(a))
    if (ni == 8) CAMX_EMB(8, true); else if (ni == 16) CAMX_EMB(16, true); else if (ni == 20) CAMX_EMB(20, true); else if (ni == 4) CAMX_EMB(4, true);
    else if (ni <= 8) CAMX_EMB(8, false); else if (ni <= 16) CAMX_EMB(16, false); else if (ni <= 24) CAMX_EMB(24, false); else CAMX_EMB(32, false);
#undef CAMX_EMB
    CAMX_LAUNCH_RET();
}

static int emb_check(const EmbArgs & a, int fmt) {
    static const int blk_bytes[FMT_COUNT] = {144, 272, 136, 82}, align[FMT_COUNT] = {16, 2, 8, 2};     // per 256 values
    if (fmt < 0 || fmt >= FMT_COUNT) return CAMX_EINVAL;
    if (!a.W || !a.toks || a.N < 256 || a.N % 256 || a.N > 8192 || a.n < 0 || a.vocab < 1) return CAMX_EINVAL;
    if (a.rb < (long)(a.N / 256 * blk_bytes[fmt])) return CAMX_EINVAL;
    if (((uintptr_t)a.W & (align[fmt] - 1)) || (a.rb & (align[fmt] - 1))) return CAMX_EINVAL;
    if (((uintptr_t)a.x & 15) || ((uintptr_t)a.xbf & 7) || ((uintptr_t)a.d & 15) || ((uintptr_t)a.nw & 15) || ((uintptr_t)a.h & 15) ||
        ((uintptr_t)a.h16 & 7) || ((uintptr_t)a.q8 & 3) || ((uintptr_t)a.err & 3)) return CAMX_EINVAL;
    return CAMX_OK;
}
static int launch_emb_fmt(const EmbArgs & a, int fmt, hipStream_t st) {
    switch (fmt) {
        case FMT_Q4_K: return launch_emb<FMT_Q4_K>(a, st);
        case FMT_Q8_0: return launch_emb<FMT_Q8_0>(a, st);
        case FMT_IQ4_XS: return launch_emb<FMT_IQ4_XS>(a, st);
        default: return launch_emb<FMT_IQ2_S>(a, st);
    }
}

// IQ4_NL rows of a per-layer-embedding feed: out[r][k] = value k of raw row inv[r] (bpr blocks of 18 bytes: f16 d, 16 bytes
// of nibbles, low nibble = value j, high = j + 16); y = d * value. One thread per four values.
__global__ void __launch_bounds__(256) ple_rows_iq4nl_k(const uint8_t * __restrict__ raw, const int * __restrict__ inv, int nuniq, int nrows,
                                                        int bpr, float * __restrict__ out, int * err) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    const int hq = bpr * 8;
    if (q >= (long)nrows * hq) return;
    const int r = (int)(q / hq), kq = (int)(q % hq), b = kq >> 3, j0 = (kq & 7) * 4;
    int u = inv[r];
    if (u < 0 || u >= nuniq) { atomicOr(err, ERR_PLE_INDEX); u = u < 0 ? 0 : nuniq - 1; }
    const uint8_t * blk = raw + (size_t)u * (size_t)(bpr * 18) + (size_t)b * 18;
    const float d = h2f_bits(*(const uint16_t *)blk);
    const uint16_t * c = (const uint16_t *)(blk + 2 + (j0 & 15));
    const uint32_t w = ((uint32_t)c[0] | ((uint32_t)c[1] << 16)) >> (j0 >= 16 ? 4 : 0);
    const f32x4 k = iq4_values(w & 0x0f0f0f0fu);
    f32x4 y; y.x = d * k.x; y.y = d * k.y; y.z = d * k.z; y.w = d * k.w;
    *(f32x4 *)(out + 4 * q) = y;
}

extern "C" {

// q3p_emb: x [n][N] fp32 = the Q4_K rows toks[i] (rb bytes per row), ids clamped to [0, vocab)
int camx_q3p_emb(const uint8_t * W, int rb, int vocab, const int32_t * toks, float * x, int N, int n, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, nullptr, N, n, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr, nullptr};
    if (!x || emb_check(a, FMT_Q4_K)) return CAMX_EINVAL;
    return launch_emb<FMT_Q4_K>(a, st);
}

// OP_OWN_EMB with its Seg fields (python/caminus/engine/k3.py:904-921, kernels/k3_own_ops.h:273-304): W = the table, a = tok, y = x
// [tokens][N], N = D, K = row bytes, work = the format's GG number (4 Q4_K, 7 IQ2_S; 3 Q8_0 as well), pad1 = 1: tok is the 64-bit key
// word of the greedy pick and the token the complement of its low half (one token), pad2 = vocab, ntask = tokens
int camx_op_own_emb(const uint8_t * W, const void * tok, float * x, int N, int K, int work, int pad1, int pad2, int tokens, hipStream_t st) {
    const int fmt = work == 4 ? FMT_Q4_K : work == 7 ? FMT_IQ2_S : work == 3 ? FMT_Q8_0 : -1;
    if (fmt < 0 || !x || (pad1 != 0 && pad1 != 1) || (pad1 && (tokens != 1 || ((uintptr_t)tok & 7)))) return CAMX_EINVAL;
    EmbArgs a = {W, K, pad2, (const int32_t *)tok, x, nullptr, N, tokens, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr, nullptr, 0, pad1};
    const int rc = emb_check(a, fmt);
    return rc ? rc : launch_emb_fmt(a, fmt, st);
}
// gather + dequant with fp32 and / or bf16 outputs; fmt 0 = Q4_K, 1 = Q8_0, 2 = IQ4_XS, 3 = IQ2_S
int camx_emb_gather(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, int N, int n, int fmt, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, xbf, N, n, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr, nullptr};
    if ((!x && !xbf) || emb_check(a, fmt)) return CAMX_EINVAL;
    return launch_emb_fmt(a, fmt, st);
}

// gather + dequant + (x += d) + RMSNorm * nw with h fp32 / fp16 / q8_1 copies, one pass per row (all outputs optional
// except that at least one is given); x receives the residual row (after the add)
int camx_emb_gather_add_rms(const uint8_t * W, long rb, int vocab, const int32_t * toks, float * x, uint16_t * xbf, const float * d,
                            const float * nw, float eps, float * h, uint16_t * h16, void * q8, int N, int n, int fmt, hipStream_t st) {
    EmbArgs a = {W, rb, vocab, toks, x, xbf, N, n, d, nw, eps, h, h16, (uint8_t *)q8, nullptr};
    if (!nw || (!x && !xbf && !h && !h16 && !q8) || emb_check(a, fmt)) return CAMX_EINVAL;
    return launch_emb_fmt(a, fmt, st);
}

// embd_rows_iq4xs: out [n][256 nblk] fp32 = the IQ4_XS rows tok[i] of table ([nvocab][136 nblk]); an id outside [0, nvocab)
// is clamped and reported as bit 1 of *err
int camx_embd_rows_iq4xs(const uint8_t * table, const int32_t * tok, int nvocab, int n, int nblk, float * out, int * err, hipStream_t st) {
    if (nblk < 1 || nblk > 32 || !out || !err) return CAMX_EINVAL;
    EmbArgs a = {table, (long)nblk * 136, nvocab, tok, out, nullptr, nblk * 256, n, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr, err};
    if (emb_check(a, FMT_IQ4_XS)) return CAMX_EINVAL;
    return launch_emb<FMT_IQ4_XS>(a, st);
}

// ple_rows_iq4nl: out [nrows][32 bpr] fp32 = the IQ4_NL rows inv[r] of raw ([nuniq][18 bpr]); an index outside [0, nuniq)
// is clamped and reported as bit 0 of *err
int camx_ple_rows_iq4nl(const uint8_t * raw, const int32_t * inv, int nuniq, int nrows, int bpr, float * out, int * err, hipStream_t st) {
    if (!raw || !inv || !out || !err || nuniq < 1 || nrows < 0 || bpr < 1 || bpr > (1 << 20) || ((uintptr_t)raw & 1) || ((uintptr_t)out & 15) ||
        ((uintptr_t)err & 3) || (long)nrows * bpr * 8 > 0x7fffffffL * 256) return CAMX_EINVAL;
    if (nrows == 0) return CAMX_OK;
    const long quads = (long)nrows * bpr * 8;
    ple_rows_iq4nl_k<<<dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st>>>(raw, inv, nuniq, nrows, bpr, out, err);
    CAMX_LAUNCH_RET();
}

}   // extern "C"
