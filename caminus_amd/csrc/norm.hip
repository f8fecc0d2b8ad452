// Residual add + RMSNorm family for gfx950: one wave64 per row, the row held in registers (128-bit loads, no LDS, no
// barrier), every copy the callers need (fp32, fp16, bf16, q8_1, row scale) written from the same registers so a row
// crosses HBM once. Replaces the reference's q3p_add_rms16 / OP_OWN_ADD_RMS16 (kernels/q3m_prefill.hip:385-415,
// kernels/k3_own_ops.h:326-383), q35p_add_rms16 (kernels/q35_prefill.hip:636-660), pf_rms_mul / OP_RMS_MUL
// (kernels/prefill_glue.hip:94-124, kernels/k3_gguf_ops.h:1233-1268), rmsnorm_f32 and residual3 (kernels/core.hip:30-61).
//
// Numeric contract: sum of squares = fmaf chain per logical thread t over elements t + 256 j, the 32-lane butterfly, the
// 8 group sums in order; scale = 1 / sqrt(tot / N + eps) with IEEE sqrt and divide; h = (x * scale) * w.
#include <type_traits>
#include "common.cuh"

enum { ADD_NONE = 0, ADD_F32_SLOTS = 1, ADD_BF16 = 2, ADD_F32_DIRECT = 3, ADD_HC = 4 };   // DIRECT: x = x + d (no 0 + d first)
// ADD_HC (pf_hc_post_rms): row q = token q / HC, stream q % HC; x = fma(d[token], 2 sigmoid(inj[q] * rs), x); gamma row q % HC

struct NormArgs {
    float * x;               // [rows][N] residual, updated in place when an addend is given
    const void * d;          // ADD_F32_SLOTS: fp32 [rows][S][N]; ADD_BF16: bf16 [rows][N]
    const float * w;         // slot weights [rows][S] or null (weights 1: acc + d)
    int S;
    const float * nw;        // gamma [wr][N]; row r uses nw[(r % wr) * N ..]
    int wr;
    float eps;
    float * h;               // optional fp32 [rows][N] (may alias x for the no-addend forms)
    uint16_t * h16;          // optional fp16 bits
    int ld16;                // h16 row stride in elements
    uint16_t * hbf;          // optional bf16 bits (to_bf16 rounding)
    uint8_t * q8;            // optional q8_1 blocks [rows][N / 32][36]
    float * scl;             // optional row scale [rows]
    int N, rows;
    const float * inj; int HC; float rs;   // ADD_HC only
    int row0;                // set by the launcher: first row of this launch (a batch may be split into a bulk launch and a tail)
    int stream;              // set by the launcher for large batches: h / h16 leave as non-temporal stores (the consumer of a decode-sized batch finds them in cache instead)
};

// EXACT: the row has exactly NI_MAX slabs, so every loop below is straight-line code: no scalar branch stands between the
// loads, which the backend then issues as one batch (with a run-time slab count each `j < ni` is a branch that loads do
// not cross, and a 4096 x 5120 launch loses 17 % to it).
// OUT != 0 is the chunk form for batches that stream from HBM: the set of copies is fixed at compile time (NORM_* bits, so
// no branch stands in the store loop either), every access is non-temporal, the requests of a row leave a short pause apart,
// and gamma waits in LDS instead of registers: GL == 1 one copy per workgroup (one gamma row for all), GL == 2 one row per
// wave (row r uses gamma row r % wr). The launcher gives these forms whole workgroups only.
enum { NORM_H = 1, NORM_H16 = 2, NORM_HBF = 4, NORM_Q8 = 8, NORM_SCL = 16 };
#define CAMX_ISSUE_GAP() do { if (OUT) { __builtin_amdgcn_sched_barrier(0); __builtin_amdgcn_s_sleep(1); __builtin_amdgcn_sched_barrier(0); } } while (0)
// SPLIT (a batch too small to fill the chip, with a q8_1 copy): a workgroup per row. Every wave loads the row and walks the same
// sum of squares (the same operations on the same values: the same bits in all four), but writes the residual and the copies of
// the slabs j = wave (mod 4) only: the serial part behind the reduction, eight q8_1 slabs for a 2048-wide row, is a quarter as long.
template <int NI_MAX, int ADD, bool EXACT, int OUT = 0, int GL = 0, bool SPLIT = false>
__global__ void __launch_bounds__(256) add_rms_rows(NormArgs a) {
    static_assert(OUT == 0 ? GL == 0 : (EXACT && !SPLIT), "the chunk form is straight-line code");
    extern __shared__ __attribute__((aligned(16))) float gsh[];
    const int lraw = threadIdx.x & 63, lane = slot_of(lraw), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int row = a.row0 + (SPLIT ? blockIdx.x : blockIdx.x * 4 + wave);
    if (!OUT && row >= a.rows) return;
    auto mine = [&](int j) { return !SPLIT || (j & 3) == wave; };
    const int N = EXACT ? NI_MAX * 256 : a.N, ni = EXACT ? NI_MAX : N >> 8;
    if (GL == 1) {
#pragma unroll
        for (int j = wave; j < NI_MAX; j += 4)      // gamma piece j (1 KiB) -> LDS in lane order; read back in slot order below
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(a.nw + 256 * j + 4 * lraw), (__attribute__((address_space(3))) void *)(gsh + 256 * j), 16, 0, 0);
    }
    if (GL == 2) {
        const float * gw2 = a.nw + (size_t)(row % a.wr) * N;
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gw2 + 256 * j + 4 * lraw), (__attribute__((address_space(3))) void *)(gsh + wave * N + 256 * j), 16, 0, 0);
    }
    float * xr = a.x + (size_t)row * N;
    f32x4 xv[NI_MAX];
    if (OUT || a.stream) {        // a batch too large to be cache resident: its rows come from HBM once, past the caches
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) { xv[j] = __builtin_nontemporal_load((const f32x4 *)(xr + 256 * j + 4 * lane)); CAMX_ISSUE_GAP(); }
    } else {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) xv[j] = *(const f32x4 *)(xr + 256 * j + 4 * lane);
    }
    // Loads never sit behind a store they might alias: the compiler cannot prove that x, d, gamma and the outputs are
    // distinct, so a load written after a store waits for everything before it (one memory round trip per slab instead of
    // one per row). Hence: every addend load, then the x stores; gamma is requested before the reduction and arrives
    // while it runs.
    const float * gw = a.nw + (size_t)(row % a.wr) * N;
    if (ADD == ADD_F32_SLOTS && a.S > 0) {
        const float * dr = (const float *)a.d + (size_t)row * a.S * N;
        const float * wr = a.w ? a.w + (size_t)row * a.S : nullptr;
        f32x4 acc[NI_MAX];
#pragma unroll
        for (int j = 0; j < NI_MAX; j++) acc[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        for (int s = 0; s < a.S; s++) {
            const float ws = wr ? wr[s] : 1.0f;
            f32x4 dv[NI_MAX];
#pragma unroll
            for (int j = 0; j < NI_MAX; j++)
                if (j < ni) { dv[j] = __builtin_nontemporal_load((const f32x4 *)(dr + (size_t)s * N + 256 * j + 4 * lane)); CAMX_ISSUE_GAP(); }
#pragma unroll
            for (int j = 0; j < NI_MAX; j++)
                if (j < ni) {
                    if (wr) {
                        acc[j].x = __builtin_fmaf(ws, dv[j].x, acc[j].x); acc[j].y = __builtin_fmaf(ws, dv[j].y, acc[j].y);
                        acc[j].z = __builtin_fmaf(ws, dv[j].z, acc[j].z); acc[j].w = __builtin_fmaf(ws, dv[j].w, acc[j].w);
                    } else acc[j] = acc[j] + dv[j];
                }
        }
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) xv[j] = xv[j] + acc[j];
    }
    if (ADD == ADD_F32_DIRECT && a.d) {
        const float * dr = (const float *)a.d + (size_t)row * N;
        // the chunk form of long rows takes the addend in two halves: 162 instead of 198 registers for a 5120-wide row, three waves per
        // SIMD instead of two (4096 x 5120: 68.0 -> 66.6 us)
        constexpr int HB = (OUT && NI_MAX > 12) ? (NI_MAX + 1) / 2 : NI_MAX;
#pragma unroll
        for (int b0 = 0; b0 < NI_MAX; b0 += HB) {
            f32x4 dv[HB];
#pragma unroll
            for (int j = 0; j < HB; j++)
                if (b0 + j < ni && b0 + j < NI_MAX) { dv[j] = __builtin_nontemporal_load((const f32x4 *)(dr + 256 * (b0 + j) + 4 * lane)); CAMX_ISSUE_GAP(); }
#pragma unroll
            for (int j = 0; j < HB; j++)
                if (b0 + j < ni && b0 + j < NI_MAX) xv[b0 + j] = xv[b0 + j] + dv[j];
            if (HB < NI_MAX) __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (ADD == ADD_BF16 && a.d) {
        const uint16_t * dr = (const uint16_t *)a.d + (size_t)row * N;
        u32x2 dv[NI_MAX];
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) { dv[j] = __builtin_nontemporal_load((const u32x2 *)(dr + 256 * j + 4 * lane)); CAMX_ISSUE_GAP(); }
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) xv[j] = xv[j] + unpack_bf16x4(dv[j]);
    }
    if (ADD == ADD_HC) {
        const float * dr = (const float *)a.d + (size_t)(row / a.HC) * N;
        f32x4 dv[NI_MAX];
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) { dv[j] = *(const f32x4 *)(dr + 256 * j + 4 * lane); CAMX_ISSUE_GAP(); }       // (plain: the HC rows of a token share it)
        const float v = a.inj[row] * a.rs;
        const float sgm = 1.0f / (1.0f + expf(-v));
        const float p = sgm * 2.0f;
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni) {
                xv[j].x = __builtin_fmaf(dv[j].x, p, xv[j].x); xv[j].y = __builtin_fmaf(dv[j].y, p, xv[j].y);
                xv[j].z = __builtin_fmaf(dv[j].z, p, xv[j].z); xv[j].w = __builtin_fmaf(dv[j].w, p, xv[j].w);
            }
    }
    f32x4 g[GL ? 1 : NI_MAX];
    if (!GL) {
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && mine(j)) g[j] = *(const f32x4 *)(gw + 256 * j + 4 * lane);
    }
    if (SPLIT) __syncthreads();                   // every wave of the row has its loads back before any of them writes (x in place; h may be x)
    if (ADD == ADD_HC || (ADD == ADD_F32_SLOTS && a.S > 0) || ((ADD == ADD_F32_DIRECT || ADD == ADD_BF16) && a.d)) {
        // the updated residual goes back to the lines it was read from
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && mine(j)) __builtin_nontemporal_store(xv[j], (f32x4 *)(xr + 256 * j + 4 * lane));
    }
    // sum of squares: logical thread 4 lane + k chains its elements in j order
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < NI_MAX; j++)
        if (j < ni) {
            ss.x = __builtin_fmaf(xv[j].x, xv[j].x, ss.x); ss.y = __builtin_fmaf(xv[j].y, xv[j].y, ss.y);
            ss.z = __builtin_fmaf(xv[j].z, xv[j].z, ss.z); ss.w = __builtin_fmaf(xv[j].w, xv[j].w, ss.w);
        }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)N + a.eps);
    if ((OUT ? (OUT & NORM_SCL) != 0 : a.scl != nullptr) && lane == 0 && (!SPLIT || wave == 0)) a.scl[row] = scale;
    if (GL) {
        __builtin_amdgcn_s_waitcnt(0x0f70);       // vmcnt(0): this wave's gamma pieces have landed in LDS (they were first in the queue)
        if (GL == 1) __syncthreads();
    }
    const float * gl = gsh + (GL == 2 ? wave * N : 0);
    // (two copies of the loop, chosen once: with the choice inside it the stores of a long row were no longer issued back to back)
    auto emit = [&](auto nt, auto redo) {
        constexpr bool NT = decltype(nt)::value, REDO = decltype(redo)::value;
        bool nan = false;
#pragma unroll
        for (int j = 0; j < NI_MAX; j++)
            if (j < ni && mine(j)) {
                const f32x4 gj = GL ? *(const f32x4 *)(gl + 256 * j + 4 * lane) : g[GL ? 0 : j];
                f32x4 t, v;
                t.x = xv[j].x * scale; t.y = xv[j].y * scale; t.z = xv[j].z * scale; t.w = xv[j].w * scale;
                v.x = t.x * gj.x; v.y = t.y * gj.y; v.z = t.z * gj.z; v.w = t.w * gj.w;
                const size_t o = (size_t)row * N + 256 * j + 4 * lane;
                if (REDO) { *(u32x2 *)(a.hbf + o) = pack_bf16x4_rne(v); continue; }
                if (OUT ? (OUT & NORM_H) != 0 : a.h != nullptr) { if (NT) __builtin_nontemporal_store(v, (f32x4 *)(a.h + o)); else *(f32x4 *)(a.h + o) = v; }
                if (OUT ? (OUT & NORM_H16) != 0 : a.h16 != nullptr) {
                    u32x2 * p16 = (u32x2 *)(a.h16 + (size_t)row * a.ld16 + 256 * j + 4 * lane);
                    // the dense line (q35p_add_rms16) stores fp16 of the last product rounded once, as the reference's binary does
                    // (kernels/q35_prefill.hip:630-635); the own line's statement is fp16 of the rounded fp32 value
                    const u32x2 pk = ADD == ADD_F32_DIRECT ? (u32x2){mul_pack_f16x2_once(t.x, gj.x, t.y, gj.y), mul_pack_f16x2_once(t.z, gj.z, t.w, gj.w)}
                                                           : pack_f16x4(v);
                    if (NT) __builtin_nontemporal_store(pk, p16); else *p16 = pk;
                }
                if (OUT ? (OUT & NORM_HBF) != 0 : a.hbf != nullptr) {
                    if (OUT) {     // the hardware convert, branch-free; a row that produced a NaN is redone below with the reference's integer rounding
                        nan |= any_nan4(v);
                        __builtin_nontemporal_store((u32x2){hw_pk_bf16(v.x, v.y), hw_pk_bf16(v.z, v.w)}, (u32x2 *)(a.hbf + o));
                    } else __builtin_nontemporal_store(pack_bf16x4_rne(v), (u32x2 *)(a.hbf + o));
                }
                if (OUT ? (OUT & NORM_Q8) != 0 : a.q8 != nullptr) q8_1_emit(v, a.q8 + ((size_t)row * (N >> 5) + 8 * j + (lane >> 3)) * 36, lane & 7);
            }
        return nan;
    };
    if (OUT) {
        const bool nan = emit(std::true_type{}, std::false_type{});
        if ((OUT & NORM_HBF) && __builtin_expect(__builtin_amdgcn_ballot_w64(nan) != 0, 0)) emit(std::true_type{}, std::true_type{});
    } else if (a.stream) emit(std::true_type{}, std::false_type{}); else emit(std::false_type{}, std::false_type{});
}
#undef CAMX_ISSUE_GAP

// Any row length (N not a multiple of 256, or longer than the register forms hold): the same tree with scalar accesses,
// x re-read for the second walk. One wave per row.
template <int ADD>
__global__ void __launch_bounds__(256) add_rms_rows_any(NormArgs a) {
    const int lane = slot_of(threadIdx.x & 63);
    const int row = a.row0 + blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (row >= a.rows) return;
    const int N = a.N;
    float * xr = a.x + (size_t)row * N;
    float ssk[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int base = 0; base < N; base += 256) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = base + 4 * lane + k;
            if (i < N) {
                float xv = xr[i];
                if (ADD == ADD_F32_SLOTS && a.S > 0) {
                    const float * dr = (const float *)a.d + (size_t)row * a.S * N;
                    const float * wr = a.w ? a.w + (size_t)row * a.S : nullptr;
                    float acc = 0.0f;
                    for (int s = 0; s < a.S; s++) acc = wr ? __builtin_fmaf(wr[s], dr[(size_t)s * N + i], acc) : acc + dr[(size_t)s * N + i];
                    xv += acc; xr[i] = xv;
                }
                if (ADD == ADD_F32_DIRECT && a.d) { xv = xv + ((const float *)a.d)[(size_t)row * N + i]; xr[i] = xv; }
                if (ADD == ADD_BF16 && a.d) { xv = xv + bf2f(((const uint16_t *)a.d)[(size_t)row * N + i]); xr[i] = xv; }
                if (ADD == ADD_HC) {
                    const float v = a.inj[row] * a.rs; const float sgm = 1.0f / (1.0f + expf(-v)); const float p = sgm * 2.0f;
                    xv = __builtin_fmaf(((const float *)a.d)[(size_t)(row / a.HC) * N + i], p, xv); xr[i] = xv;
                }
                ssk[k] = __builtin_fmaf(xv, xv, ssk[k]);
            }
        }
    }
    const f32x4 ss = {ssk[0], ssk[1], ssk[2], ssk[3]};
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)N + a.eps);
    if (a.scl && lane == 0) a.scl[row] = scale;
    const float * gw = a.nw + (size_t)(row % a.wr) * N;
    // (a lane re-reads only elements it stored itself: program order covers it)
    for (int base = 0; base < N; base += 256) {
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        float vk[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = base + 4 * lane + k;
            vk[k] = 0.0f;
            if (i < N) {
                vk[k] = (xr[i] * scale) * gw[i];
                const size_t o = (size_t)row * N + i;
                if (a.h) a.h[o] = vk[k];
                if (a.h16) a.h16[(size_t)row * a.ld16 + i] = ADD == ADD_F32_DIRECT ? (uint16_t)mul_pack_f16x2_once(xr[i] * scale, gw[i], 0.0f, 0.0f) : f2h_bits(vk[k]);
                if (a.hbf) a.hbf[o] = to_bf16(vk[k]);
            }
        }
        v.x = vk[0]; v.y = vk[1]; v.z = vk[2]; v.w = vk[3];
        if (a.q8 && base + 4 * (lane & ~7) < N)    // N % 32 == 0 is checked on the host when a q8 copy is asked for
            q8_1_emit(v, a.q8 + ((size_t)row * (N >> 5) + (base >> 5) + (lane >> 3)) * 36, lane & 7);
    }
}

// The chunk form with a row divided over W waves of the workgroup (W = 4: a workgroup per row; W = 2: two rows): a wave takes the NS
// slabs part NS .. of its row (N = 256 NS W), so a quarter or half of the row sits in a wave, W times as many waves are in flight, and each
// stores its part of the residual as soon as its own loads are back. The sum of squares keeps its order: logical thread 4 lane + k chains
// its elements slab by slab, so the lane's four partial sums go from wave to wave through LDS (part p continues where part p - 1 stopped)
// and the last part forms the row's total with the same tree. Gamma comes straight into registers (a wave needs NS slabs of it).
template <int NS, int W, int ADD, int OUT>
__global__ void __launch_bounds__(256) add_rms_rows_div(NormArgs a) {
    static_assert(ADD == ADD_NONE || ADD == ADD_F32_SLOTS || ADD == ADD_F32_DIRECT, "the addends of the row kernels");
    constexpr int N = NS * W * 256, RPW = 4 / W;
    __shared__ __attribute__((aligned(16))) float chain[RPW][256];
    __shared__ float totsh[RPW];
    const int lraw = threadIdx.x & 63, lane = slot_of(lraw), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = wave / W, part = wave % W;
    const int row = a.row0 + blockIdx.x * RPW + rw;
    const int e0 = part * (NS * 256) + 4 * lane;                        // this lane's first element of the row
    float * xr = a.x + (size_t)row * N + e0;
    f32x4 xv[NS];
#pragma unroll
    for (int j = 0; j < NS; j++) xv[j] = __builtin_nontemporal_load((const f32x4 *)(xr + 256 * j));
    bool added = false;
    if (ADD == ADD_F32_SLOTS && a.S > 0) {
        const float * dr = (const float *)a.d + (size_t)row * a.S * N + e0;
        const float * wr = a.w ? a.w + (size_t)row * a.S : nullptr;
        f32x4 acc[NS];
#pragma unroll
        for (int j = 0; j < NS; j++) acc[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        for (int s = 0; s < a.S; s++) {
            const float ws = wr ? wr[s] : 1.0f;
            f32x4 dv[NS];
#pragma unroll
            for (int j = 0; j < NS; j++) dv[j] = __builtin_nontemporal_load((const f32x4 *)(dr + (size_t)s * N + 256 * j));
#pragma unroll
            for (int j = 0; j < NS; j++) {
                if (wr) {
                    acc[j].x = __builtin_fmaf(ws, dv[j].x, acc[j].x); acc[j].y = __builtin_fmaf(ws, dv[j].y, acc[j].y);
                    acc[j].z = __builtin_fmaf(ws, dv[j].z, acc[j].z); acc[j].w = __builtin_fmaf(ws, dv[j].w, acc[j].w);
                } else acc[j] = acc[j] + dv[j];
            }
        }
#pragma unroll
        for (int j = 0; j < NS; j++) xv[j] = xv[j] + acc[j];
        added = true;
    }
    if (ADD == ADD_F32_DIRECT && a.d) {
        const float * dr = (const float *)a.d + (size_t)row * N + e0;
        f32x4 dv[NS];
#pragma unroll
        for (int j = 0; j < NS; j++) dv[j] = __builtin_nontemporal_load((const f32x4 *)(dr + 256 * j));
#pragma unroll
        for (int j = 0; j < NS; j++) xv[j] = xv[j] + dv[j];
        added = true;
    }
    const float * gw = a.nw + (size_t)(row % a.wr) * N + e0;
    f32x4 g[NS];
#pragma unroll
    for (int j = 0; j < NS; j++) g[j] = *(const f32x4 *)(gw + 256 * j);
    if (added) {
#pragma unroll
        for (int j = 0; j < NS; j++) __builtin_nontemporal_store(xv[j], (f32x4 *)(xr + 256 * j));
    }
#pragma unroll
    for (int p = 0; p < W; p++) {
        if (part == p) {
            f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
            if (p) ss = *(const f32x4 *)(chain[rw] + 4 * lraw);
#pragma unroll
            for (int j = 0; j < NS; j++) {
                ss.x = __builtin_fmaf(xv[j].x, xv[j].x, ss.x); ss.y = __builtin_fmaf(xv[j].y, xv[j].y, ss.y);
                ss.z = __builtin_fmaf(xv[j].z, xv[j].z, ss.z); ss.w = __builtin_fmaf(xv[j].w, xv[j].w, ss.w);
            }
            if (p < W - 1) *(f32x4 *)(chain[rw] + 4 * lraw) = ss;
            else { const float tot = wave_groups_in_order(group32_sum(ss)); if (lraw == 0) totsh[rw] = tot; }
        }
        __syncthreads();
    }
    const float scale = rsqrt_exact(totsh[rw] / (float)N + a.eps);
    if ((OUT & NORM_SCL) && part == 0 && lane == 0) a.scl[row] = scale;
    auto emit = [&](auto redo) {
        constexpr bool REDO = decltype(redo)::value;
        bool nan = false;
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const f32x4 gj = g[j];
            f32x4 t, v;
            t.x = xv[j].x * scale; t.y = xv[j].y * scale; t.z = xv[j].z * scale; t.w = xv[j].w * scale;
            v.x = t.x * gj.x; v.y = t.y * gj.y; v.z = t.z * gj.z; v.w = t.w * gj.w;
            const size_t o = (size_t)row * N + e0 + 256 * j;
            if (REDO) { *(u32x2 *)(a.hbf + o) = pack_bf16x4_rne(v); continue; }
            if (OUT & NORM_H) __builtin_nontemporal_store(v, (f32x4 *)(a.h + o));
            if (OUT & NORM_H16) {
                u32x2 * p16 = (u32x2 *)(a.h16 + (size_t)row * a.ld16 + e0 + 256 * j);
                const u32x2 pk = ADD == ADD_F32_DIRECT ? (u32x2){mul_pack_f16x2_once(t.x, gj.x, t.y, gj.y), mul_pack_f16x2_once(t.z, gj.z, t.w, gj.w)}
                                                       : pack_f16x4(v);
                __builtin_nontemporal_store(pk, p16);
            }
            if (OUT & NORM_HBF) {
                nan |= any_nan4(v);
                __builtin_nontemporal_store((u32x2){hw_pk_bf16(v.x, v.y), hw_pk_bf16(v.z, v.w)}, (u32x2 *)(a.hbf + o));
            }
            if (OUT & NORM_Q8) q8_1_emit(v, a.q8 + ((size_t)row * (N >> 5) + 8 * (part * NS + j) + (lane >> 3)) * 36, lane & 7);
        }
        return nan;
    };
    const bool nan = emit(std::false_type{});
    if ((OUT & NORM_HBF) && __builtin_expect(__builtin_amdgcn_ballot_w64(nan) != 0, 0)) emit(std::true_type{});
}
template <int ADD, int OUT>
static int launch_norm_div(const NormArgs & a, hipStream_t st) {
    if constexpr (ADD == ADD_NONE || ADD == ADD_F32_SLOTS || ADD == ADD_F32_DIRECT) {
        // Measured against the wave-per-row chunk form (cold lines): with a q8_1 copy 23.1 -> 22.2 us at 4096 x 2048 (the encode behind the
        // reduction is a quarter as long per wave), 2560-wide rows over two waves 24.3 -> 23.4 us at 8192 rows, and 1.5 - 2 % from 16384 rows on;
        // q3p_add_rms16 at 4096 x 2048 is slower this way (26.7 -> 28.3 us) and keeps the wave per row.
        const int ni = a.N >> 8;
        if (!((OUT & NORM_Q8) || ni == 10 || a.rows >= 16384)) return 0;
        const int w = ni == 10 ? 2 : 4, rpw = 4 / w, rows = a.rows - a.rows % rpw;
        if (rows == 0) return 0;
        NormArgs b = a; b.rows = rows;
        const dim3 grid(rows / rpw), block(256);
        switch (ni) {
        case 4: add_rms_rows_div<1, 4, ADD, OUT><<<grid, block, 0, st>>>(b); return rows;
        case 8: add_rms_rows_div<2, 4, ADD, OUT><<<grid, block, 0, st>>>(b); return rows;
        case 10: add_rms_rows_div<5, 2, ADD, OUT><<<grid, block, 0, st>>>(b); return rows;
        case 16: add_rms_rows_div<4, 4, ADD, OUT><<<grid, block, 0, st>>>(b); return rows;
        case 20: add_rms_rows_div<5, 4, ADD, OUT><<<grid, block, 0, st>>>(b); return rows;
        }
    }
    return 0;
}

// The chunk form of add_rms_rows for one set of copies, if the launch fits it: returns the rows it took (whole workgroups).
template <int ADD, int OUT>
static int launch_norm_chunk(const NormArgs & a, hipStream_t st) {
    const int rows = a.rows & ~3, ni = a.N >> 8, gl = a.wr == 1 ? 1 : 2;
    if (gl == 2 && a.N > 2560) return 0;          // (a gamma row per wave: 4 N floats of LDS per workgroup)
    const dim3 grid(rows / 4), block(256);
    const size_t lds = (size_t)(gl == 1 ? 1 : 4) * a.N * sizeof(float);
    NormArgs b = a; b.rows = rows;
    switch (ni) {
#define CAMX_NORM_CHUNK(NI) case NI: \
        if (gl == 1) add_rms_rows<NI, ADD, true, OUT, 1><<<grid, block, lds, st>>>(b); \
        else if constexpr (ADD == ADD_NONE || ADD == ADD_HC) { if constexpr (NI <= 10) add_rms_rows<NI, ADD, true, OUT, 2><<<grid, block, lds, st>>>(b); } \
        else return 0; \
        return rows;
        CAMX_NORM_CHUNK(4) CAMX_NORM_CHUNK(8) CAMX_NORM_CHUNK(10) CAMX_NORM_CHUNK(16) CAMX_NORM_CHUNK(20)
#undef CAMX_NORM_CHUNK
    }
    return 0;
}

// CHUNK_OUTS: the sets of copies (NORM_* masks) this entry point's prefill callers ask for; a batch that streams from HBM
// with one of them runs the chunk form, anything else the general one.
template <int ADD, int... CHUNK_OUTS>
static int launch_norm(const NormArgs & a0, hipStream_t st) {
    if (a0.rows <= 0) return CAMX_OK;
    NormArgs a = a0;
    a.row0 = 0;
    a.stream = (long)a.rows * a.N >= (1L << 20);
    const int ni = a.N >> 8;
    const bool vec = (a.N & 255) == 0 && ni <= 32 && (a.ld16 & 3) == 0 &&
                     ((uintptr_t)a.x & 15) == 0 && ((uintptr_t)a.nw & 15) == 0 && ((uintptr_t)a.d & 15) == 0 && ((uintptr_t)a.h & 15) == 0 &&
                     ((uintptr_t)a.h16 & 7) == 0 && ((uintptr_t)a.hbf & 7) == 0 && ((uintptr_t)a.q8 & 3) == 0;
    if (vec && a.stream && a.rows >= 1024 && (ADD == ADD_NONE || ADD == ADD_HC || a.d)) {
        const int mask = (a.h ? NORM_H : 0) | (a.h16 ? NORM_H16 : 0) | (a.hbf ? NORM_HBF : 0) | (a.q8 ? NORM_Q8 : 0) | (a.scl ? NORM_SCL : 0);
        int done = 0;
        (void)((mask == CHUNK_OUTS && ((done = launch_norm_div<ADD, CHUNK_OUTS>(a, st)) || (done = launch_norm_chunk<ADD, CHUNK_OUTS>(a, st)), true)) || ...);
        if (done) {
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess || done == a.rows) return (int)e;
            a.row0 = done;                        // the last rows % 4 rows
        }
    }
    const dim3 block(256);
    // a workgroup per row: up to 1024 rows when a q8_1 copy follows the reduction, else up to 256 (5120-wide rows: 7.3 us against 8.7 for
    // 256 cold rows, equal from 512 rows on; 2048-wide rows: within 4 % either way)
    if (vec && a.rows <= (a.q8 ? 1024 : 256)) {
        const dim3 grid(a.rows);
        switch (ni) {
#define CAMX_NORM_SPLIT(NI) case NI: add_rms_rows<NI, ADD, true, 0, 0, true><<<grid, block, 0, st>>>(a); CAMX_LAUNCH_RET();
            CAMX_NORM_SPLIT(4) CAMX_NORM_SPLIT(8) CAMX_NORM_SPLIT(10) CAMX_NORM_SPLIT(16) CAMX_NORM_SPLIT(20)
#undef CAMX_NORM_SPLIT
        }
    }
    const dim3 grid((a.rows - a.row0 + 3) / 4);
    if (!vec) add_rms_rows_any<ADD><<<grid, block, 0, st>>>(a);
    else switch (ni) {
#define CAMX_NORM_EXACT(NI) case NI: add_rms_rows<NI, ADD, true><<<grid, block, 0, st>>>(a); break;
        CAMX_NORM_EXACT(1) CAMX_NORM_EXACT(2) CAMX_NORM_EXACT(3) CAMX_NORM_EXACT(4) CAMX_NORM_EXACT(5) CAMX_NORM_EXACT(6) CAMX_NORM_EXACT(7)
        CAMX_NORM_EXACT(8) CAMX_NORM_EXACT(10) CAMX_NORM_EXACT(12) CAMX_NORM_EXACT(14) CAMX_NORM_EXACT(16) CAMX_NORM_EXACT(20)
        CAMX_NORM_EXACT(24) CAMX_NORM_EXACT(28) CAMX_NORM_EXACT(32)
#undef CAMX_NORM_EXACT
        default:
            if (ni <= 16) add_rms_rows<16, ADD, false><<<grid, block, 0, st>>>(a);
            else if (ni <= 24) add_rms_rows<24, ADD, false><<<grid, block, 0, st>>>(a);
            else add_rms_rows<32, ADD, false><<<grid, block, 0, st>>>(a);
    }
    CAMX_LAUNCH_RET();
}

// ---- the dense bf16 prefill form at chunk sizes: x += bf16 addend, RMSNorm, bf16 copy -------------------------------------------
// One wave per row as above, written for this one job so that nothing stands between the loads: gamma goes straight to LDS
// (one copy per workgroup, no registers, first in the queue), then every x and addend load of the row is issued, a short
// pause apart, before the first dependent instruction; the residual goes back as soon as it is summed, and the bf16 rows are
// packed by the hardware convert and stored without a branch in the loop (a row that produced a NaN is redone with the
// reference's integer rounding, which has no NaN case). A wave's reads and writes are two separate bursts: HBM serves a read
// burst and a write burst faster than an interleaved stream. rows % 4 == 0 (no partial workgroup).
template <int NI>
__global__ void __launch_bounds__(256) add_rms_bf16_chunk(float * __restrict__ x, const uint16_t * __restrict__ d, const float * __restrict__ nw, float eps,
                                                          uint16_t * __restrict__ hbf) {
    extern __shared__ __attribute__((aligned(16))) float gsh[];
    constexpr int N = NI * 256;
    const int lraw = threadIdx.x & 63, lane = slot_of(lraw), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t row = (size_t)blockIdx.x * 4 + wave;
#pragma unroll
    for (int j = wave; j < NI; j += 4)      // gamma piece j (1 KiB) -> LDS in lane order; read back in slot order below
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(nw + 256 * j + 4 * lraw), (__attribute__((address_space(3))) void *)(gsh + 256 * j), 16, 0, 0);
    float * xr = x + row * N;
    const uint16_t * dr = d + row * N;
    f32x4 xv[NI]; u32x2 dv[NI > 12 ? (NI + 1) / 2 : NI];
    // (the pause between requests: 4096 waves that each fire 40 requests at once measured 2 % slower than the same requests a few dozen cycles apart)
#define CAMX_ISSUE_GAP() do { __builtin_amdgcn_sched_barrier(0); __builtin_amdgcn_s_sleep(1); __builtin_amdgcn_sched_barrier(0); } while (0)
#pragma unroll
    for (int j = 0; j < NI; j++) { xv[j] = __builtin_nontemporal_load((const f32x4 *)(xr + 256 * j + 4 * lane)); CAMX_ISSUE_GAP(); }
    // (long rows take the addend in two halves: fewer registers, one more wave per SIMD; 4096 x 5120: 44.1 -> 43.5 us, three parts: 44.6)
    constexpr int HB = NI > 12 ? (NI + 1) / 2 : NI;
#pragma unroll
    for (int b0 = 0; b0 < NI; b0 += HB) {
#pragma unroll
        for (int j = b0; j < b0 + HB && j < NI; j++) { dv[j - b0] = __builtin_nontemporal_load((const u32x2 *)(dr + 256 * j + 4 * lane)); CAMX_ISSUE_GAP(); }
#pragma unroll
        for (int j = b0; j < b0 + HB && j < NI; j++) xv[j] = xv[j] + unpack_bf16x4(dv[j - b0]);
        if (HB < NI) __builtin_amdgcn_sched_barrier(0);
    }
#undef CAMX_ISSUE_GAP
#pragma unroll
    for (int j = 0; j < NI; j++) __builtin_nontemporal_store(xv[j], (f32x4 *)(xr + 256 * j + 4 * lane));
    f32x4 ss = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < NI; j++) {
        ss.x = __builtin_fmaf(xv[j].x, xv[j].x, ss.x); ss.y = __builtin_fmaf(xv[j].y, xv[j].y, ss.y);
        ss.z = __builtin_fmaf(xv[j].z, xv[j].z, ss.z); ss.w = __builtin_fmaf(xv[j].w, xv[j].w, ss.w);
    }
    const float tot = wave_groups_in_order(group32_sum(ss));
    const float scale = rsqrt_exact(tot / (float)N + eps);
    __builtin_amdgcn_s_waitcnt(0x0f70);       // vmcnt(0): this wave's gamma pieces have landed in LDS (they were first in the queue)
    __syncthreads();
    uint16_t * hr = hbf + row * N;
    bool nan = false;
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const f32x4 g = *(const f32x4 *)(gsh + 256 * j + 4 * lane);
        f32x4 v;
        v.x = (xv[j].x * scale) * g.x; v.y = (xv[j].y * scale) * g.y; v.z = (xv[j].z * scale) * g.z; v.w = (xv[j].w * scale) * g.w;
        nan |= any_nan4(v);
        const u32x2 pk = {hw_pk_bf16(v.x, v.y), hw_pk_bf16(v.z, v.w)};
        __builtin_nontemporal_store(pk, (u32x2 *)(hr + 256 * j + 4 * lane));
    }
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(nan) != 0, 0)) {
#pragma unroll
        for (int j = 0; j < NI; j++) {          // (unrolled: a register array cannot be indexed by a loop counter)
            const f32x4 g = *(const f32x4 *)(gsh + 256 * j + 4 * lane);
            f32x4 v;
            v.x = (xv[j].x * scale) * g.x; v.y = (xv[j].y * scale) * g.y; v.z = (xv[j].z * scale) * g.z; v.w = (xv[j].w * scale) * g.w;
            *(u32x2 *)(hr + 256 * j + 4 * lane) = pack_bf16x4_rne(v);
        }
    }
}
// Takes the first n - n % 4 rows when the chunk form applies (an addend, a bf16 copy and no fp32 copy, a chunk of at least 1024
// rows of 256 NI values for the NI below, 16-byte aligned) and returns how many rows it took.
static int launch_add_rms_bf16_chunk(float * x, const uint16_t * d, const float * nw, float eps, uint16_t * hbf, int N, int n, hipStream_t st) {
    if (!d || !hbf || n < 1024 || (N & 255) || (((uintptr_t)x | (uintptr_t)d | (uintptr_t)nw | (uintptr_t)hbf) & 15)) return 0;
    const int rows = n & ~3;
    const dim3 grid(rows / 4), block(256);
    switch (N >> 8) {
#define CAMX_CHUNK(NI) case NI: add_rms_bf16_chunk<NI><<<grid, block, NI * 1024, st>>>(x, d, nw, eps, hbf); return rows;
        CAMX_CHUNK(4) CAMX_CHUNK(6) CAMX_CHUNK(8) CAMX_CHUNK(10) CAMX_CHUNK(12) CAMX_CHUNK(14) CAMX_CHUNK(16) CAMX_CHUNK(20) CAMX_CHUNK(24) CAMX_CHUNK(28) CAMX_CHUNK(32)
#undef CAMX_CHUNK
    }
    return 0;
}

extern "C" {

int camx_q3p_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h,
                       uint16_t * h16, int N, int n, hipStream_t st) {
    if (N < 256 || N % 256 || N > 2048 || S < 0 || S > 8 || n < 0 || !x || !nw || !h16 || (S > 0 && !d)) return CAMX_EINVAL;
    NormArgs a = {x, d, w, d ? S : 0, nw, 1, eps, h, h16, N, nullptr, nullptr, nullptr, N, n, nullptr, 1, 0.0f};
    return launch_norm<ADD_F32_SLOTS, NORM_H16, NORM_H | NORM_H16>(a, st);
}

// OP_OWN_ADD_RMS16 with its Seg fields (python/caminus/engine/k3.py:881-902): W = nw, gs = w, a = d, asum = h, y = x, rs = eps, N,
// K = the fp16 copy's token stride (elements, >= N), pad1 = S, aux = h16, tokens = the tape's T
// OP_OWN_ADD_RMS16 as the dense line's modules run it (kernels/k3_q35_ops.h:79-130): any row length N = 256 NI up to 65536, one addend with
// weight 1 (S = 1) or none, h always written, the fp16 copy rounded once from the last product (camx_q35p_add_rms16's arithmetic) at token stride K
int camx_op_q35_add_rms16(float * x, const float * d, int S, const float * nw, float eps, float * h, uint16_t * h16, int N, int K, int tokens, hipStream_t st) {
    if (N < 256 || N % 256 || N > 65536 || K < N || S < 0 || S > 1 || tokens < 0 || !x || !nw || !h || !h16 || (S > 0 && !d)) return CAMX_EINVAL;
    NormArgs a = {x, S ? d : nullptr, nullptr, 0, nw, 1, eps, h, h16, K, nullptr, nullptr, nullptr, N, tokens, nullptr, 1, 0.0f};
    return launch_norm<ADD_F32_DIRECT, NORM_H | NORM_H16>(a, st);
}
int camx_op_own_add_rms16(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h, uint16_t * h16,
                          int N, int K, int tokens, hipStream_t st) {
    if (N < 256 || N % 256 || N > 65536 || K < N || S < 0 || S > 8 || tokens < 0 || !x || !nw || !h16 || (S > 0 && !d)) return CAMX_EINVAL;
    if (N > 2048) return w ? CAMX_EINVAL : camx_op_q35_add_rms16(x, d, S, nw, eps, h, h16, N, K, tokens, st);      // only the dense line's modules have rows this long
    NormArgs a = {x, d, w, d ? S : 0, nw, 1, eps, h, h16, K, nullptr, nullptr, nullptr, N, tokens, nullptr, 1, 0.0f};
    return launch_norm<ADD_F32_SLOTS, NORM_H16, NORM_H | NORM_H16>(a, st);
}

int camx_q35p_add_rms16(float * x, const float * d, const float * nw, float eps, float * h, uint16_t * h16, int N, int n, hipStream_t st) {
    if (N < 256 || N % 256 || N > 65536 || n < 0 || !x || !nw || !h || !h16) return CAMX_EINVAL;
    NormArgs a = {x, d, nullptr, 0, nw, 1, eps, h, h16, N, nullptr, nullptr, nullptr, N, n, nullptr, 1, 0.0f};
    return launch_norm<ADD_F32_DIRECT, NORM_H | NORM_H16>(a, st);
}

int camx_add_rms_q8_1(float * x, const float * d, const float * w, int S, const float * nw, float eps, float * h,
                      uint16_t * h16, uint8_t * q8, int N, int n, hipStream_t st) {
    if (N < 32 || N % 32 || S < 0 || S > 8 || n < 0 || !x || !nw || (S > 0 && !d)) return CAMX_EINVAL;
    NormArgs a = {x, d, w, d ? S : 0, nw, 1, eps, h, h16, N, nullptr, q8, nullptr, N, n, nullptr, 1, 0.0f};
    return launch_norm<ADD_F32_SLOTS, NORM_Q8, NORM_H | NORM_Q8, NORM_H | NORM_H16 | NORM_Q8>(a, st);
}

int camx_add_rms_bf16(float * x, const uint16_t * d, const float * nw, float eps, float * h, uint16_t * hbf, int N, int n, hipStream_t st) {
    if (N < 1 || n < 0 || !x || !nw) return CAMX_EINVAL;
    if (!h) {
        const int done = launch_add_rms_bf16_chunk(x, d, nw, eps, hbf, N, n, st);
        if (done) {
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess || done == n) return (int)e;
            x += (size_t)done * N; d += (size_t)done * N; hbf += (size_t)done * N; n -= done;     // the last n % 4 rows
        }
    }
    NormArgs a = {x, d, nullptr, 0, nw, 1, eps, h, nullptr, N, hbf, nullptr, nullptr, N, n, nullptr, 1, 0.0f};
    return launch_norm<ADD_BF16>(a, st);
}

int camx_pf_rms_mul(const float * x, const float * w, float * y, uint16_t * ybf, float * scl, int R, int wr, float eps, int K, hipStream_t st) {
    if (K < 1 || R < 0 || wr < 1 || !x || !w) return CAMX_EINVAL;
    NormArgs a = {(float *)x, nullptr, nullptr, 0, w, wr, eps, y, nullptr, K, ybf, nullptr, scl, K, R, nullptr, 1, 0.0f};
    return launch_norm<ADD_NONE, NORM_H, NORM_HBF | NORM_SCL, NORM_HBF>(a, st);
}

int camx_op_rms_mul(const float * x, const float * w, float * y, uint8_t * q8, int R, int wr, int K, float eps, hipStream_t st) {
    if (K < 1 || R < 0 || wr < 1 || !x || !w || (q8 && K % 32)) return CAMX_EINVAL;
    NormArgs a = {(float *)x, nullptr, nullptr, 0, w, wr, eps, y, nullptr, K, nullptr, q8, nullptr, K, R, nullptr, 1, 0.0f};
    return launch_norm<ADD_NONE, NORM_H, NORM_H | NORM_Q8>(a, st);
}

// pf_hc_post_rms: res [T * HC][N] updated in place, then its norm with w [HC][N]; xn, xnbf, scl optional
int camx_pf_hc_post_rms(const float * b, const float * inj, float * res, const float * w, float * xn, uint16_t * xnbf, float * scl, int T, int HC,
                        float rs, float eps, int N, hipStream_t st) {
    if (!b || !inj || !res || !w || T < 0 || HC < 1 || N < 1 || (long)T * HC > 0x7fffffffL) return CAMX_EINVAL;
    NormArgs a = {res, b, nullptr, 0, w, HC, eps, xn, nullptr, N, xnbf, nullptr, scl, N, T * HC, inj, HC, rs};
    return launch_norm<ADD_HC, NORM_HBF | NORM_SCL, NORM_HBF>(a, st);
}

int camx_rmsnorm_f32(const float * x, const float * w, float * out, int D, float eps, int rows, hipStream_t st) {
    if (D < 1 || rows < 0 || !x || !w || !out) return CAMX_EINVAL;
    NormArgs a = {(float *)x, nullptr, nullptr, 0, w, 1, eps, out, nullptr, D, nullptr, nullptr, nullptr, D, rows, nullptr, 1, 0.0f};
    return launch_norm<ADD_NONE, NORM_H>(a, st);
}

}   // extern "C"
