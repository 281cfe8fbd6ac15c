// Quantized matmul for prefill chunks (m > 32) on the tiled layout: the only shape of this path that
// is a dense contraction, so this kernel is priced against the MFMA peak, not HBM.
//
// MFMA shape.  v_mfma_f32_32x32x16_f16: on MI355X it sustains about 2.1 PFLOP/s in a register-only
// loop, the 16x16x32 form only about 1.4, so the GEMM uses 32x32 tiles (the skinny kernel keeps
// 16x16x32 because its limit is HBM, not the matrix pipe).
//
// Tiling.  Workgroup tile 256 (m) x 96 (n), 4 waves stacked along m; wave tile 64 x 96 = 2 x 3 MFMA
// tiles (96 accumulator registers).  Activations arrive prepared in 32-row A-fragment order
// (act_prep32_kernel) and are copied global -> LDS by global_load_lds_dwordx4 (no registers, no
// ds_write), 64 columns (4 operand steps) per stage, three stage buffers, loads issued two stages
// ahead, one barrier per stage.  Weights do NOT go through LDS: each wave loads the packed bytes of
// its six row tiles straight into registers and unpacks them with the and_or / pk_fma arithmetic of
// the skinny kernel; one unpacked B operand (32 rows x 16 columns) feeds two MFMAs.
//   B operand of 32 rows = two 16-row tiles: lane l = n32 + 32 * g32 reads row r = n32 % 16 of tile
//   n32 / 16 and takes the tile's lane slots 2 * g32 and 2 * g32 + 1 (columns 128 * g32 .. +127 of
//   the super-block), 16 operand steps of 8 columns each; the activation fragments use the same order.
//
// Block scales.  The skinny kernel keeps the weights as exact integers and applies d / dmin in f32 on
// each tile result; with 96 accumulators that would need a second accumulator set.  Here the f16
// super-block scale is folded into the packed-f16 constants instead: B = nibble * f16(d * sc) (two
// roundings of 2^-12 relative), and the "- dmin * m" term is one extra MFMA per super-block against
// the activation sub-block sums with B = -f16(dmin * m).  Against the f32 matmul on dequantized
// weights this costs about 3e-4 relative L2 (bar: 1e-3).  The dispatcher only uses this kernel while
// 1024 * d * sc stays inside f16.
#include <hip/hip_ext.h>

#include "layout.h"
#include "mfma_common.h"

namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr uint32_t kMagic1024 = 0x64006400u;  // 1024.0: a nibble in mantissa bits 0..3 reads as 1024 + n
constexpr uint32_t kMagic64 = 0x54005400u;    // 64.0:   a nibble in mantissa bits 4..7 reads as 64 + n
constexpr int BM = 256, BN = 96;              // workgroup tile
constexpr int WM = 2, WN = 3;                 // 32x32 MFMA tiles per wave: 64 x 96
constexpr int STAGE_STEPS = 4;                // operand steps (16 columns each) per LDS stage
constexpr int STAGE_BYTES = STAGE_STEPS * (BM / 32) * 1024;  // 32 KiB
constexpr int NBUF = 3;

__device__ inline _Float16 h_from_bits(uint32_t bits16) {
    const uint16_t u = (uint16_t)bits16;
    _Float16 h;
    __builtin_memcpy(&h, &u, 2);
    return h;
}

__device__ inline float16v mfma32x32x16(half8v a, half8v b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// wait until at most N of this wave's vector-memory operations are outstanding (they retire in order)
template <int N> __device__ inline void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// LDS reads of the activation fragments are written as asm with hand-placed waits: the compiler counts an
// LDS-DMA copy as both a memory and an LDS event and from then on waits for lgkmcnt(0) at every LDS use, which
// would serialise each read with the MFMAs that follow it.
template <int OFF> __device__ inline half8v lds_read128(uint32_t addr) {
    half8v v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
// wait until at most N LDS reads are outstanding; the two fragments pass through the statement so that their
// users cannot be scheduled ahead of it
template <int N> __device__ inline void lds_wait_pin(half8v &a0, half8v &a1) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a0), "+v"(a1) : "n"(N));
}

// packed bytes of one 32-row group for one super-block: two lane slots of a tile + that row's header
struct BRegs { uint4v qa[2], qb[2], hd; };

__device__ inline BRegs b_load(const uint8_t *__restrict__ tile, int r, int g32) {
    using F = TiledFmt<TURQ_Q4_K>;
    BRegs t;
#pragma unroll
    for (int s = 0; s < 2; s++) {
        const int slot = r + 16 * (2 * g32 + s);
        t.qa[s] = *(const uint4v *)(tile + F::kQA + 16 * slot);
        t.qb[s] = *(const uint4v *)(tile + F::kQB + 16 * slot);
    }
    t.hd = *(const uint4v *)(tile + F::kHDR + 16 * r);
    return t;
}

// constants of the lane's four sub-blocks u = 2 * slot + half (sub-block 4 * g32 + u of the super-block)
struct BConsts {
    half2v s[4], c1[4], c2[4];  // d*sc, -1024*d*sc, -64*d*sc (both halves equal)
    half8v bmin;                // -(dmin*m_u) twice each, against the (hi, lo) sums fragment
};

__device__ inline BConsts b_consts(uint4v hd, int g32) {
    // 24-bit groups of lane slots 2*g32 and 2*g32+1 inside the 96-bit field hd.y, hd.z, hd.w
    // (both candidates are computed and selected: a divergent branch would cost more than the two shifts)
    const uint32_t g0a = hd.y, g0b = __builtin_amdgcn_alignbit(hd.w, hd.z, 16);
    const uint32_t g1a = __builtin_amdgcn_alignbit(hd.z, hd.y, 24), g1b = hd.w >> 8;
    const uint32_t msk = (uint32_t)-g32;  // all ones for the upper lane half
    const uint32_t G0 = (g0a & ~msk) | (g0b & msk);
    const uint32_t G1 = (g1a & ~msk) | (g1b & msk);
    const half2v k1024 = splat2((_Float16)1024.0f);
    const half2v dd = splat2(h_from_bits(hd.x & 0xFFFFu));
    const half2v dm = splat2((_Float16)(-(float)h_from_bits(hd.x >> 16)));
    BConsts c;
    half2v mn[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
        const uint32_t G = s ? G1 : G0;
        const half2v sc = as_half2((G & 0x3Fu) | ((G << 4) & 0x003F0000u) | kMagic1024) - k1024;
        mn[s] = (as_half2(((G >> 6) & 0x3Fu) | ((G >> 2) & 0x003F0000u) | kMagic1024) - k1024) * dm;
        const half2v dsc = sc * dd;  // (d*sc of half 0, d*sc of half 1), rounded to f16
        c.s[2 * s] = splat2(dsc.x);
        c.s[2 * s + 1] = splat2(dsc.y);
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
        c.c1[u] = c.s[u] * splat2((_Float16)-1024.0f);
        c.c2[u] = c.s[u] * splat2((_Float16)-64.0f);
    }
    c.bmin = half8v{mn[0].x, mn[0].x, mn[0].y, mn[0].y, mn[1].x, mn[1].x, mn[1].y, mn[1].y};
    return c;
}

__device__ inline half8v q4_operand(uint32_t w, half2v s, half2v c1, half2v c2) {
    const uint32_t w8 = w >> 8;
    return make_half8(pk_fma(and_or_h2(w, 0x000F000Fu, kMagic1024), s, c1), pk_fma(and_or_h2(w, 0x00F000F0u, kMagic64), s, c2),
                      pk_fma(and_or_h2(w8, 0x000F000Fu, kMagic1024), s, c1), pk_fma(and_or_h2(w8, 0x00F000F0u, kMagic64), s, c2));
}

// frags: 32-row fragments, 1 KiB block index (mt * ntc + b) * 17 + q
__global__ void __launch_bounds__(256) gemm_q4k_kernel(const uint8_t *__restrict__ w, int64_t n, int64_t k,
                                                       const uint8_t *__restrict__ frags, int64_t m, void *__restrict__ y,
                                                       int yt, int64_t ldy, const float *__restrict__ bias, int nblocks_n,
                                                       int nblocks_m) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // NBUF stages of 32 KiB
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n32 = lane & 31, g32 = lane >> 5;
    const int r16 = n32 & 15, tsel = n32 >> 4;
    // Workgroups of one XCD (blockIdx % 8) get consecutive logical ids and the m-blocks of one n-block are
    // consecutive in that order: the packed weights they share stay in that XCD's L2.
    const int nwg = nblocks_n * nblocks_m;
    int lid = blockIdx.x;
    if ((nwg & 7) == 0) lid = (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3);
    const int nb = lid / nblocks_m, mb = lid - nb * nblocks_m;
    const int64_t ntc = turq_tile_cols(k);
    const int64_t mtiles = (m + 31) / 32;
    const int64_t nrt = turq_tile_rows(n);
    constexpr int TB = TiledFmt<TURQ_Q4_K>::kTileBytes;

    // the 16-row tile this lane reads for each of the wave's three 32-row groups (clamped at the end)
    const uint8_t *wrow[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        int64_t rt = (int64_t)nb * (BN / 16) + 2 * j + tsel;
        rt = rt < nrt ? rt : nrt - 1;
        wrow[j] = w + rt * ntc * TB;
    }

    float16v acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Stage s = 5 * b + ks.  ks < 4: operand steps 4ks .. 4ks+3 of super-block b for the 8 m-tiles of the
    // workgroup (32 blocks of 1 KiB; wave w copies step 4ks + w for all 8 m-tiles); ks == 4: the sums step
    // (8 blocks, wave w copies m-tiles 2w, 2w+1).  All index arithmetic is 32-bit and wave-uniform.
    const int nstages = (int)ntc * 5;
    const int ntc_i = (int)ntc;
    // 1 KiB block index of (m-tile c of this workgroup, super-block 0, step 0); tiles past the end re-read the
    // last valid one (their rows are never stored) so that every wave always issues the same number of loads,
    // which the vmcnt bookkeeping below relies on
    int mt_blk[8];
#pragma unroll
    for (int c = 0; c < 8; c++) {
        int64_t mtg = (int64_t)mb * (BM / 32) + c;
        mtg = mtg < mtiles ? mtg : mtiles - 1;
        mt_blk[c] = (int)(mtg * ntc * 17);
    }
    const uint32_t lane_off = 16u * (uint32_t)lane;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    auto issue_one = [&](int blk1k, int dst_off) {
        const uint8_t *src = frags + ((size_t)blk1k << 10);  // wave-uniform
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + lane_off),
                                         (__attribute__((address_space(3))) void *)(lds + dst_off), 16, 0, 0);
    };
    // issue stage (b, ks) into buffer `buf`
    auto stage_issue = [&](int b, int ks, int buf) {
        const int base = buf * STAGE_BYTES;
        if (ks < 4) {
            const int q = 4 * ks + wave;
#pragma unroll
            for (int c = 0; c < 8; c++) issue_one(mt_blk[c] + b * 17 + q, base + ((wave * 8 + c) << 10));
        } else {
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int mt = 2 * wave + c;
                int blk = 0;
#pragma unroll
                for (int t = 0; t < 8; t++) blk = (t == mt) ? mt_blk[t] : blk;  // uniform select, no dynamic indexing
                issue_one(blk + b * 17 + 16, base + (mt << 10));
            }
        }
    };

    BRegs wt[WN], wnext[WN];
    BConsts cs[WN], cs_next[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) wt[j] = b_load(wrow[j], r16, g32);
#pragma unroll
    for (int j = 0; j < WN; j++) cs[j] = b_consts(wt[j].hd, g32);
    stage_issue(0, 0, 0);
    stage_issue(0, 1, 1);
    int buf = 0;          // buffer of the stage being computed
    int ib = 0, iks = 2;  // (super-block, ks) of the next stage to issue, i.e. stage s + 2
    int ibuf = 2;

    for (int b = 0; b < ntc_i; b++) {
#pragma unroll
        for (int ks = 0; ks < 5; ks++) {  // fully unrolled: ks selects registers at compile time
            // Stage s was issued two stages ago.  Loads retire in order, so "at most as many outstanding as the
            // newest stage issued" means stage s (and the weight loads before it) have landed.
            // (Past the last stage the issue below repeats the last super-block into a buffer nobody reads any
            // more, which keeps these counts the same for every stage and the loop free of branches.)
            if (ks == 3) wait_vmcnt<2>(); else wait_vmcnt<8>();   // the sums stage has 2 loads per wave
            // plain s_barrier: __syncthreads() would also drain the loads that are meant to stay in flight
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // now stage s is visible to all waves and nobody reads buffer (s + 2) % 3 any more
            static_assert(WM == 2, "fragment double buffering below is written for two m-tiles per wave");
            const uint32_t abase = lds_base + (uint32_t)(buf * STAGE_BYTES + (wave * WM << 10)) + lane_off;
            half8v af[2][WM];  // [step parity][m-tile]
            af[0][0] = lds_read128<0>(abase);
            af[0][1] = lds_read128<1024>(abase);
            if (ks == 2) {
                // the next super-block's weights were issued before stage s + 1's copies, so the wait of the
                // previous stage has covered them
#pragma unroll
                for (int j = 0; j < WN; j++) cs_next[j] = b_consts(wnext[j].hd, g32);
            }
            if (ks == 0) {
                const int bn = b + 1 < ntc_i ? b + 1 : b;  // last super-block: harmless re-read
#pragma unroll
                for (int j = 0; j < WN; j++) wnext[j] = b_load(wrow[j] + (int64_t)bn * TB, r16, g32);
            }
            stage_issue(ib < ntc_i ? ib : ntc_i - 1, iks, ibuf);
            iks = iks == 4 ? 0 : iks + 1;
            ib += iks == 0 ? 1 : 0;
            ibuf = ibuf == NBUF - 1 ? 0 : ibuf + 1;
            if (ks < 4) {
#pragma unroll
                for (int st = 0; st < STAGE_STEPS; st++) {
                    const int cur = st & 1, nxt = cur ^ 1;
                    if (st + 1 < STAGE_STEPS) {  // next step's activation fragments come in while this step computes
                        const uint32_t an = abase + (uint32_t)((st + 1) * (BM / 32) << 10);
                        af[nxt][0] = lds_read128<0>(an);
                        af[nxt][1] = lds_read128<1024>(an);
                        lds_wait_pin<2>(af[cur][0], af[cur][1]);
                    } else {
                        lds_wait_pin<0>(af[cur][0], af[cur][1]);
                    }
                    const int q = 4 * ks + st;            // operand step 0..15: slot q >> 3, dword q & 7
                    const int slot = q >> 3, dw = q & 7;
                    const int u = 2 * slot + (dw >> 2);   // sub-block index among the lane's four
                    half8v bop[WN];
#pragma unroll
                    for (int j = 0; j < WN; j++) {
                        const uint4v src = dw < 4 ? wt[j].qa[slot] : wt[j].qb[slot];
                        const uint32_t wd = (dw & 3) == 0 ? src.x : (dw & 3) == 1 ? src.y : (dw & 3) == 2 ? src.z : src.w;
                        bop[j] = q4_operand(wd, cs[j].s[u], cs[j].c1[u], cs[j].c2[u]);
                    }
#pragma unroll
                    for (int i = 0; i < WM; i++)
#pragma unroll
                        for (int j = 0; j < WN; j++) acc[i][j] = mfma32x32x16(af[cur][i], bop[j], acc[i][j]);
                }
            } else {
                // "- dmin * m" term against the sub-block sums; then the prefetched weights take over
                lds_wait_pin<0>(af[0][0], af[0][1]);
#pragma unroll
                for (int i = 0; i < WM; i++)
#pragma unroll
                    for (int j = 0; j < WN; j++) acc[i][j] = mfma32x32x16(af[0][i], cs[j].bmin, acc[i][j]);
#pragma unroll
                for (int j = 0; j < WN; j++) {
                    wt[j] = wnext[j];
                    cs[j] = cs_next[j];
                }
            }
            buf = buf == NBUF - 1 ? 0 : buf + 1;
        }
    }
    wait_vmcnt<0>();  // the two trailing dummy stages must not outlive the workgroup's LDS

    // 32x32 result: lane (n32, g32), register e holds row 8 * (e / 4) + 4 * g32 + e % 4 of column n32
#pragma unroll
    for (int j = 0; j < WN; j++) {
        const int64_t col = (int64_t)nb * BN + 32 * j + n32;
        if (col >= n) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < WM; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int64_t row = (int64_t)mb * BM + (wave * WM + i) * 32 + 8 * (e >> 2) + 4 * g32 + (e & 3);
                if (row < m) {
                    const float v = acc[i][j][e] + bv;
                    if (yt == TURQ_ACT_F32) turq_store_out<TURQ_ACT_F32>(y, row * ldy + col, v);
                    else if (yt == TURQ_ACT_BF16) turq_store_out<TURQ_ACT_BF16>(y, row * ldy + col, v);
                    else turq_store_out<TURQ_ACT_F16>(y, row * ldy + col, v);
                }
            }
    }
}

}  // namespace

// frags: activations prepared by turq_launch_act_prep32 for all m rows
hipError_t turq_launch_gemm_mfma(int dtype, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y,
                                 int y_dtype, int64_t ldy, const float *bias, hipStream_t stream, hipEvent_t ev_start,
                                 hipEvent_t ev_stop) {
    if (n == 0 || m == 0) return hipSuccess;
    if (dtype != TURQ_Q4_K) return hipErrorInvalidValue;
    static const hipError_t attr = hipFuncSetAttribute((const void *)gemm_q4k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       NBUF * STAGE_BYTES);
    if (attr != hipSuccess) return attr;
    const int nbn = (int)((n + BN - 1) / BN), nbm = (int)((m + BM - 1) / BM);
    const dim3 grid((unsigned)(nbn * nbm)), block(256);
    const unsigned lds_bytes = NBUF * STAGE_BYTES;
    if (ev_start) {
        hipExtLaunchKernelGGL(gemm_q4k_kernel, grid, block, lds_bytes, stream, ev_start, ev_stop, 0, (const uint8_t *)w, n, k,
                              (const uint8_t *)frags, m, y, y_dtype, ldy, bias, nbn, nbm);
    } else {
        gemm_q4k_kernel<<<grid, block, lds_bytes, stream>>>((const uint8_t *)w, n, k, (const uint8_t *)frags, m, y, y_dtype, ldy,
                                                            bias, nbn, nbm);
    }
    return hipGetLastError();
}
