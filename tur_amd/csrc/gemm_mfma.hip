// Quantized matmul for prefill chunks (m > 32) on the tiled layout: the only shape of this path that
// is a dense contraction, so this kernel is priced against the MFMA peak, not HBM.
//
// MFMA shape.  v_mfma_f32_32x32x16_f16: on MI355X it sustains about 2.1 PFLOP/s in a register-only
// loop, the 16x16x32 form only about 1.4, so the GEMM uses 32x32 tiles (the skinny kernel keeps
// 16x16x32 because its limit is HBM, not the matrix pipe).  Vector ALU work of the same SIMD is NOT
// hidden under the MFMAs (about 2 cycles per VALU instruction on top of the 32 of an MFMA, also with
// two waves per SIMD), so the loop is written to spend as few other instructions as it can.
//
// Tiling.  A workgroup is 4 waves and takes 128 rows of m.  Q4_K: tile 128 (m) x 192 (n), waves as 2 x 2, wave tile
// 64 x 96 = 2 x 3 MFMA tiles (96 accumulator registers).  The activations are the expensive operand here (2 bytes per
// element against 0.56 for the weights), hence the wide n.  Q5_K / Q6_K, whose unpack is two to three times as long: tile
// 128 x 128 with the waves as 1 x 4, wave tile 128 x 32 = 4 x 1 MFMA tiles, so that every weight is unpacked by one wave
// instead of two (the 2 x 2 grid is 18 % slower for Q6_K, 7 % for Q5_K).
//
// Everything reaches the LDS by global_load_lds_dwordx4 (no registers, no ds_write):
//   * activations, prepared in 32-row A-fragment order (act_prep32_kernel), 64 columns (4 operand
//     steps) of the workgroup's 4 m-tiles per stage = 16 KiB, ring of 4 stages; stage s + 4 is issued
//     as soon as every wave is done with stage s;
//   * the packed weight tiles of the workgroup's 12 row tiles, 27 KiB per super-block, ring of 3,
//     issued two super-blocks ahead in four groups, because they come from HBM and loads of one wave
//     retire in order: a late weight load delays every younger activation load of that wave;
//   * the activation sub-block sums of the 4 m-tiles, 4 KiB per super-block, ring of 2.
// Every wave issues the same number of copies at every stage boundary (4 + 2, + 1 sums block at the
// first of a super-block; past the end they repeat the last super-block into buffers nobody reads),
// so the "at most N copies outstanding" waits are compile-time constants.  There is one barrier per
// stage; it sits before the last operand step of the previous stage, so that the first LDS reads of
// the new stage run under those MFMAs.
//
// LDS reads and the copies are written as asm with hand-placed waits: the compiler counts an LDS-DMA
// copy both as a memory and as an LDS event and from then on waits for lgkmcnt(0) at every LDS use,
// and __syncthreads() would drain the copies that are meant to stay in flight.
//
//   B operand of 32 rows = two 16-row tiles: lane l = n32 + 32 * g32 reads row r = n32 % 16 of tile
//   n32 / 16 and takes the tile's lane slots 2 * g32 and 2 * g32 + 1 (columns 128 * g32 .. +127 of
//   the super-block), 16 operand steps of 8 columns each; the activation fragments use the same order.
//   Stage ks of a super-block is the lane's sub-block ks: one 16-byte LDS read per 32-row tile.
//
// Block scales.  The skinny kernel keeps the weights as exact integers and applies d / dmin in f32 on
// each tile result; with 96 accumulators that would need a second accumulator set.  Here the f16
// super-block scale is folded into the packed-f16 constants instead: B = nibble * f16(d * sc) (two
// roundings of 2^-12 relative), and the "- dmin * m" term is one extra MFMA per super-block against
// the activation sub-block sums with B = -f16(dmin * m).  Against the f32 matmul on dequantized
// weights this costs about 3e-4 relative L2 (bar: 1e-3).  The dispatcher only uses this kernel while
// 1024 * d * sc stays inside f16.
//
// Formats.  Q4_K as above.  Q5_K adds the fifth bit from the tile's
// high-bit plane with one rotate and one v_and_or_b32 per packed register; Q6_K builds the whole 6-bit value in
// the mantissa of 256.0 (low nibble at bits 2..5, high field rotated onto bits 6..7) and needs no sums term.  Their
// tiles are larger (2816 / 3360 bytes), so their workgroup is 128 x 128 to keep three super-blocks of weights in the LDS.  Q8_0 (4352-byte tiles, f16 block scales, no sums term): 128 x 64, wave tile 2 x 1.
//
// Launches that would leave CUs idle.  Three further forms of the same loop, chosen per launch by the rules at the end of this
// file: every tile's super-blocks shared out over several workgroups that meet in device memory (SK); the low tile with eight
// waves as two groups on alternate super-blocks that meet in the LDS (KG = 2); and up to four weights of one format in one
// launch (GemmGroup), the n-blocks dealt out to them in order.
//
// Results leave through the LDS (free after the main loop): each wave transposes its 64 x 96 tile so
// that a lane stores 16 contiguous bytes and a row segment is 192 (bf16, f16) or 384 (f32) bytes.
#include <hip/hip_ext.h>

#include <cstdlib>
#include <type_traits>
#include <utility>

#include "layout.h"
#include "mfma_common.h"

#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as a clobber on purpose

namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr uint32_t kMagic1024 = 0x64006400u;  // 1024.0: a nibble in mantissa bits 0..3 reads as 1024 + n
constexpr uint32_t kMagic64 = 0x54005400u;    // 64.0:   a nibble in mantissa bits 4..7 reads as 64 + n
constexpr uint32_t kMagic256 = 0x5C005C00u;   // 256.0:  a 6-bit value in mantissa bits 2..7 reads as 256 + q
constexpr int kCoherent = 16;                 // cache policy of buffer loads and stores that other XCDs must see: sc1, as device-scope atomics carry
// lanes whose value is no finite number, or too large for the output type: one vector compare, the OR runs on the scalar unit
__device__ inline uint64_t note_mask(float v, float lim) { return __builtin_amdgcn_ballot_w64(!(__builtin_fabsf(v) < lim)); }
// A workgroup is 4 waves and covers 128 rows of m (4 m-tiles of 32): as 2 x 2 waves with 2 m-tiles each (WGM = 2), or as
// 1 x 4 waves that all take the 4 m-tiles (WGM = 1: every weight is unpacked by ONE wave instead of two, at twice the
// activation reads per wave; for the formats whose unpack is long)
constexpr int BM = 128;
constexpr int MT = BM / 32;                   // m-tiles per workgroup; wave w copies m-tile w
constexpr int A_STAGE = MT * 4 * 1024;        // [m-tile][step] blocks of 1 KiB
constexpr int NA = 4;                         // stage ring; 4 stages per super-block, so stage ks lives in buffer ks
constexpr int NW = 3;                         // weight ring (super-blocks)
constexpr int S_BYTES = MT * 1024;
constexpr int NS = 2;
static_assert(MT == 4, "the copy and read schedules below are written for this shape");

// 32x32 tiles per wave along n in the 2 x 2 wave grid, by format (the per-format pieces are further down)
template <int DT> struct GFmtWN;
template <> struct GFmtWN<TURQ_Q4_K> { static constexpr int value = 3; };
template <> struct GFmtWN<TURQ_Q5_K> { static constexpr int value = 2; };
template <> struct GFmtWN<TURQ_Q6_K> { static constexpr int value = 2; };
template <> struct GFmtWN<TURQ_Q8_0> { static constexpr int value = 1; };

// geometry that depends on the format and the wave grid: WGM x WGN waves, WM x WN 32x32 tiles per wave
// WGM_ = 3 is the WIDE form of the 1 x 4 grid: two 32x32 tiles per wave along n (workgroup tile 128 x 256), which halves the
// activation bytes a launch pulls through the L2 per flop; to fit the LDS its rings are two deep (activation stages and
// weight super-blocks alike) and the weights of a super-block are requested in two halves, at the last boundary of the
// super-block before the previous one and at the first of the previous one.
template <int DT, int WGM_> struct Geo {
    // WGM_ = 4 is the LOW form for launches that would leave CUs idle: 64 rows of m (two m-tiles) by 128 of n, four waves of
    // 64 x 32, i.e. twice the workgroups of the 128 x 128 tile; it uses the wide form's two-deep rings and copy schedule.
    static_assert(WGM_ >= 1 && WGM_ <= 4, "wave grid 2 x 2, 1 x 4, or 1 x 4 with the wide or the low tile");
    static constexpr bool LOW = WGM_ == 4;
    static constexpr bool WIDE = WGM_ == 3 || LOW;                 // (the ring and copy schedule, not the width)
    static constexpr int GMT = LOW ? 2 : MT;                       // m-tiles per workgroup
    static constexpr int GBM = GMT * 32;
    static constexpr int GA_STAGE = GMT * 4 * 1024;
    static constexpr int WGM = WIDE ? 1 : WGM_, WGN = 4 / WGM, WM = GMT / WGM;
    static constexpr int WN = WGM_ == 2 ? GFmtWN<DT>::value : (WGM_ == 3 ? 2 : 1);  // 1 x 4 waves: 128 (wide: 256) rows of n
    static constexpr int RA = WIDE ? 2 : NA, RW = WIDE ? 2 : NW;               // ring depths
    static constexpr int BN = WGN * WN * 32;
    static constexpr int NT16 = BN / 16;                           // 16-row weight tiles per workgroup
    static constexpr int TB = TiledFmt<DT>::kTileBytes;
    static constexpr int W_BYTES = NT16 * TB;
    static constexpr int W_CHUNKS = (W_BYTES + 1023) / 1024;       // copies of 1 KiB; the last may be partial
    static constexpr int W_STRIDE = W_CHUNKS * 1024;               // ring stride: a partial last copy lands in padding
    static constexpr int CPW = 2 * ((W_CHUNKS + 7) / 8);           // wide form: weight copies per wave and super-block (even)
    static constexpr int A_OFF = 0, W_OFF = RA * GA_STAGE, S_OFF = W_OFF + RW * W_STRIDE;
    static constexpr int OUT_PITCH = WN * 32 + 8;                  // floats per staged result row: rows r and r + 4 land 32 banks apart
    static_assert(WIDE || W_CHUNKS <= 32, "weight copies: two per wave and group");
    static_assert(!WIDE || (CPW % 2 == 0 && CPW <= 24), "wide form: two halves of CPW / 2 copies per wave");
};

// Up to kMaxGroup weights of one format and one k against the same activation fragments in ONE launch (gate and up of an MLP):
// the n-blocks [first[i], first[i + 1]) of the launch belong to weight i.  One launch over the rows of both fills the rounds
// over the CUs better than two (and picks its tile for the rows of both).
constexpr int kMaxGroup = 4;
struct GemmGroup {
    const uint8_t *w[kMaxGroup];
    void *y[kMaxGroup];
    const float *bias[kMaxGroup];
    int64_t n[kMaxGroup], ldy[kMaxGroup];
    float wscale[kMaxGroup];  // per tensor: see the kernel
    int first[kMaxGroup];
    int count;
};

template <int... I, typename F> __device__ inline void static_for_impl(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): loop indices usable as template arguments
template <int N, typename F> __device__ inline void static_for(F &&f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

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
// wait until at most N of this wave's LDS reads are outstanding
template <int N> __device__ inline void wait_lds() { asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory"); }
// a value read by lds_read128 may be used only after a wait; passing it through an (empty) volatile
// statement placed after that wait keeps its users from being scheduled ahead of the wait (the value it yields is a new one
// to the compiler, so no copy made earlier can stand in for it).  What the compiler could still do is copy or spill the
// register between the read and the wait; the build walks the device assembly of this file and fails if any instruction
// touches the destination of an LDS read before the wait that covers it, or if a kernel here spills (check_lds_waits.py).
template <typename T> __device__ inline void pin(T &v) { asm volatile("" : "+v"(v)); }

template <int OFF, typename T> __device__ inline void lds_read128(T &dst, uint32_t addr) {
    static_assert(sizeof(T) == 16 && OFF >= 0 && OFF < 65536, "one ds_read_b128");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

template <int OFF> __device__ inline void lds_read64(uint2v &dst, uint32_t addr) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF> __device__ inline void lds_read32(uint32_t &dst, uint32_t addr) {
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF> __device__ inline void lds_read16(uint32_t &dst, uint32_t addr) {
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

// 64 lanes x 16 bytes, global -> LDS.  The instruction offset applies to both sides: lane l copies
// sbase[voff_l + IMM .. + 15] to LDS byte lds_addr + IMM + 16 * l.
template <int IMM> __device__ inline void dma_set(uint32_t voff, const uint8_t *sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_addr), "n"(IMM)
                 : "memory", "m0");
}
// same LDS base (m0) as the preceding dma_set of this wave
template <int IMM> __device__ inline void dma_more(uint32_t voff, const uint8_t *sbase) {
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
}

// 64-bit address arithmetic may run on the vector ALU even when every input is uniform; the copies take
// their base address in scalar registers
__device__ inline const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(((uint64_t)hi << 32) | lo);
}

template <int I> __device__ inline uint32_t word_of(uint4v v) { return I == 0 ? v.x : I == 1 ? v.y : I == 2 ? v.z : v.w; }

__device__ inline uint32_t pack_bf16x2(float a, float b) { return turq_f2bf_x2(a, b); }
__device__ inline uint32_t pack_f16x2(float a, float b) {
    const half2v h{(_Float16)a, (_Float16)b};
    return as_u32(h);
}

// ---- per-format pieces -------------------------------------------------------------------------------------
// A lane (n32, g32) of a 32-row B tile works on row r16 = n32 % 16 of 16-row tile n32 / 16 and on that tile's lane
// slots 2 g32 and 2 g32 + 1 (64 columns each).  Stage ks of a super-block covers the 32 columns of half (ks & 1) of
// slot 2 g32 + (ks >> 1): operand steps i = 4 (ks & 1) + st, st = 0..3, of that slot.
//   Stage   what a lane reads from the LDS for one stage and one 32-row tile (NSTG reads)
//   Hdr     what it reads once per super-block (NHDR reads)
//   Consts  packed-f16 constants derived from Hdr
//   `tile` is the LDS address of the lane's 16-row tile in the weight ring entry.
template <int DT> struct GFmt;

struct K4Consts {
    half2v s[4], s16[4], c1[4], c2[4];  // per sub-block u = ks: d*sc, d*sc/16, -1024*d*sc, -64*d*sc (both halves equal)
    half8v bmin;                        // -(dmin*m_u) twice each, against the (hi, lo) sums fragment
};

// constants of the lane's four sub-blocks u (sub-block 4 * g32 + u of the super-block) from a Q4_K / Q5_K header row
__device__ inline K4Consts k4_consts(uint4v hd, int g32, _Float16 ws) {
    // 24-bit groups of lane slots 2*g32 and 2*g32+1 inside the 96-bit field hd.y, hd.z, hd.w
    // (both candidates are computed and selected: a divergent branch would cost more than the two shifts)
    const uint32_t g0a = hd.y, g0b = __builtin_amdgcn_alignbit(hd.w, hd.z, 16);
    const uint32_t g1a = __builtin_amdgcn_alignbit(hd.z, hd.y, 24), g1b = hd.w >> 8;
    const uint32_t msk = (uint32_t)-g32;  // all ones for the upper lane half
    const uint32_t G0 = (g0a & ~msk) | (g0b & msk);
    const uint32_t G1 = (g1a & ~msk) | (g1b & msk);
    const half2v k1024 = splat2((_Float16)1024.0f);
    const half2v dd = splat2(h_from_bits(hd.x & 0xFFFFu) * ws);  // ws is a power of two: exact
    const half2v dm = splat2(-h_from_bits(hd.x >> 16) * ws);
    K4Consts c;
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
        c.s16[u] = c.s[u] * splat2((_Float16)0.0625f);
        c.c1[u] = c.s[u] * splat2((_Float16)-1024.0f);
        c.c2[u] = c.s[u] * splat2((_Float16)-64.0f);
    }
    c.bmin = half8v{mn[0].x, mn[0].x, mn[0].y, mn[0].y, mn[1].x, mn[1].x, mn[1].y, mn[1].y};
    return c;
}

template <> struct GFmt<TURQ_Q4_K> {
    using F = TiledFmt<TURQ_Q4_K>;
    static constexpr int NSTG = 1;
    static constexpr bool SUMS = true;
    struct Stage { uint4v q; };
    struct Hdr { uint4v hd; };
    using Consts = K4Consts;
    struct Addr { uint32_t q, h; };
    __device__ static Addr addr(uint32_t tile, int r16, int g32) {
        return Addr{tile + 16u * (uint32_t)(r16 + 32 * g32), tile + (uint32_t)F::kHDR + 16u * (uint32_t)r16};
    }
    // OFF = byte offset of the n-tile inside the ring entry (compile time)
    template <int KS, int OFF> __device__ static void read_stage(Stage &st, const Addr &a, uint32_t ring) {
        lds_read128<OFF + (KS & 1) * 1024 + (KS >> 1) * 256>(st.q, a.q + ring);
    }
    template <int OFF> __device__ static void read_hdr(Hdr &h, const Addr &a, uint32_t ring) { lds_read128<OFF>(h.hd, a.h + ring); }
    __device__ static void pin_stage(Stage &st) { pin(st.q); }
    __device__ static void pin_hdr(Hdr &h) { pin(h.hd); }
    __device__ static Consts consts(const Hdr &h, int g32, _Float16 ws) { return k4_consts(h.hd, g32, ws); }
    __device__ static half8v bmin(const Consts &c) { return c.bmin; }
    template <int KS, int ST> __device__ static half8v operand(const Stage &st, const Consts &c) {
        const uint32_t w = word_of<ST>(st.q), w8 = w >> 8;
        return make_half8(pk_fma(and_or_asm_h2(w, 0x000F000Fu, kMagic1024), c.s[KS], c.c1[KS]), pk_fma(and_or_asm_h2(w, 0x00F000F0u, kMagic64), c.s[KS], c.c2[KS]),
                          pk_fma(and_or_asm_h2(w8, 0x000F000Fu, kMagic1024), c.s[KS], c.c1[KS]),
                          pk_fma(and_or_asm_h2(w8, 0x00F000F0u, kMagic64), c.s[KS], c.c2[KS]));
    }
};

template <> struct GFmt<TURQ_Q5_K> {
    using F = TiledFmt<TURQ_Q5_K>;
    static constexpr int NSTG = 2;
    static constexpr bool SUMS = true;
    struct Stage { uint4v q; uint2v hh; };
    struct Hdr { uint4v hd; };
    using Consts = K4Consts;
    struct Addr { uint32_t q, hh, h; };
    __device__ static Addr addr(uint32_t tile, int r16, int g32) {
        return Addr{tile + 16u * (uint32_t)(r16 + 32 * g32), tile + (uint32_t)F::kQH + 8u * (uint32_t)(r16 + 32 * g32),
                    tile + (uint32_t)F::kHDR + 16u * (uint32_t)r16};
    }
    template <int KS, int OFF> __device__ static void read_stage(Stage &st, const Addr &a, uint32_t ring) {
        lds_read128<OFF + (KS & 1) * 1024 + (KS >> 1) * 256>(st.q, a.q + ring);
        lds_read64<OFF + (KS >> 1) * 128>(st.hh, a.hh + ring);  // the two high-bit dwords of the lane slot
    }
    template <int OFF> __device__ static void read_hdr(Hdr &h, const Addr &a, uint32_t ring) { lds_read128<OFF>(h.hd, a.h + ring); }
    __device__ static void pin_stage(Stage &st) { pin(st.q); pin(st.hh); }
    __device__ static void pin_hdr(Hdr &h) { pin(h.hd); }
    __device__ static Consts consts(const Hdr &h, int g32, _Float16 ws) { return k4_consts(h.hd, g32, ws); }
    __device__ static half8v bmin(const Consts &c) { return c.bmin; }
    template <int KS, int ST> __device__ static half8v operand(const Stage &st, const Consts &c) {
        // step i of the slot; with v = 4 i + t the packed register t, u = v >> 1: its two high bits sit in H0 (even t) at
        // bits (4 + u, 20 + u) or in H1 (odd t) at bits (8 + u, 24 + u): a rotate right by u puts them on bit 4 / 20
        // (+16 on a nibble at bits 0..3) or bit 8 / 24 (+16 on a nibble at bits 4..7 read with 16 units per step)
        constexpr uint32_t u0 = 2 * (4 * (KS & 1) + ST);
        const uint32_t w = word_of<ST>(st.q), w8 = w >> 8;
        uint32_t t0 = and_or_asm(w, 0x000F000Fu, kMagic1024);
        uint32_t t1 = and_or_asm(w, 0x00F000F0u, kMagic1024);
        uint32_t t2 = and_or_asm(w8, 0x000F000Fu, kMagic1024);
        uint32_t t3 = and_or_asm(w8, 0x00F000F0u, kMagic1024);
        t0 = and_or_asm(rotr32(st.hh.x, u0), 0x00100010u, t0);
        t1 = and_or_asm(rotr32(st.hh.y, u0), 0x01000100u, t1);
        t2 = and_or_asm(rotr32(st.hh.x, u0 + 1), 0x00100010u, t2);
        t3 = and_or_asm(rotr32(st.hh.y, u0 + 1), 0x01000100u, t3);
        return make_half8(pk_fma(as_half2(t0), c.s[KS], c.c1[KS]), pk_fma(as_half2(t1), c.s16[KS], c.c2[KS]),
                          pk_fma(as_half2(t2), c.s[KS], c.c1[KS]), pk_fma(as_half2(t3), c.s16[KS], c.c2[KS]));
    }
};

template <> struct GFmt<TURQ_Q6_K> {
    using F = TiledFmt<TURQ_Q6_K>;
    static constexpr int NSTG = 2;
    static constexpr bool SUMS = false;
    struct Stage { uint4v ql, qh; };
    struct Hdr { uint32_t sc0, sc1, d16; };  // the four int8 scales of lane slots 2 g32 and 2 g32 + 1; the row's d
    struct Consts { half2v s[8]; };          // per 16-column group of the lane's 128 columns: d*sc, rounded to f16
    struct Addr { uint32_t q, qh, sc, d; };
    __device__ static Addr addr(uint32_t tile, int r16, int g32) {
        const uint32_t slot = (uint32_t)(r16 + 32 * g32);
        return Addr{tile + 16u * slot, tile + (uint32_t)F::kQH + 16u * slot, tile + (uint32_t)F::kSC + 4u * slot,
                    tile + (uint32_t)F::kD + 2u * (uint32_t)r16};
    }
    template <int KS, int OFF> __device__ static void read_stage(Stage &st, const Addr &a, uint32_t ring) {
        lds_read128<OFF + (KS & 1) * 1024 + (KS >> 1) * 256>(st.ql, a.q + ring);
        lds_read128<OFF + (KS >> 1) * 256>(st.qh, a.qh + ring);  // all 64 high fields of the lane slot
    }
    template <int OFF> __device__ static void read_hdr(Hdr &h, const Addr &a, uint32_t ring) {
        lds_read32<OFF>(h.sc0, a.sc + ring);
        lds_read32<OFF + 64>(h.sc1, a.sc + ring);
        lds_read16<OFF>(h.d16, a.d + ring);
    }
    __device__ static void pin_stage(Stage &st) { pin(st.ql); pin(st.qh); }
    __device__ static void pin_hdr(Hdr &h) { pin(h.sc0); pin(h.sc1); pin(h.d16); }
    __device__ static Consts consts(const Hdr &h, int, _Float16 ws) {
        const float d = (float)h_from_bits(h.d16) * (float)ws;
        Consts c;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int sc = (int)(int8_t)((i < 4 ? h.sc0 : h.sc1) >> (8 * (i & 3)));
            const _Float16 s = (_Float16)(d * (float)sc);
            c.s[i] = splat2(s);
        }
        return c;
    }
    __device__ static half8v bmin(const Consts &c) { return half8v{}; }
    template <int KS, int ST> __device__ static half8v operand(const Stage &st, const Consts &c) {
        // step i = 4 (KS & 1) + ST of the slot: low nibbles of register t at bits 2 + 4 t (and + 16), high fields at bits
        // 6 + 8 (i & 1) + 2 t (and + 16) of high dword i >> 1; scale group i >> 1 of the slot
        constexpr int i = 4 * (KS & 1) + ST;
        constexpr int grp = 4 * (KS >> 1) + (i >> 1);
        const uint32_t wl = word_of<ST>(st.ql);
        const uint32_t wh = word_of<(i >> 1)>(st.qh);
        half2v r[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t lo = and_or_asm(t == 0 ? wl : rotr32(wl, 4 * t), 0x003C003Cu, kMagic256);
            const uint32_t hi_src = (8 * (i & 1) + 2 * t) == 0 ? wh : rotr32(wh, (uint32_t)(8 * (i & 1) + 2 * t));
            // (256 + q) - 288 = q - 32 exactly, then one rounding in the product; a fused form would need the constant
            // -288 * d * sc, which f16 cannot hold exactly (288 is not a power of two)
            r[t] = (as_half2(and_or_asm(hi_src, 0x00C000C0u, lo)) - splat2((_Float16)288.0f)) * c.s[grp];
        }
        return make_half8(r[0], r[1], r[2], r[3]);
    }
};

// Q8_0: the tile holds 8 blocks of 32 columns in four planes (plane i = blocks 2 i, 2 i + 1); stage ks is plane ks.  The lane
// reads its two lane slots (2 g32, 2 g32 + 1: 8 bytes per block each) and takes, per block, first the 8 columns of the one,
// then of the other: operand step st of the stage is block 2 ks + st / 2, slot st % 2 (the Q8_0 order of act_prep32_kernel).
// Bytes are q + 128 (tiled layout), read as 1024 + 128 + q in the mantissa of 1024.0; (t - 1152) is q exactly and q * d is
// rounded once.  The tiles are 4352 bytes: wave tile 2 x 1 (workgroup 128 x 64) keeps three super-blocks in the LDS.
template <> struct GFmt<TURQ_Q8_0> {
    using F = TiledFmt<TURQ_Q8_0>;
    static constexpr int NSTG = 2;
    static constexpr bool SUMS = false;
    struct Stage { uint4v a, b; };     // lane slots 2 g32 and 2 g32 + 1 of the plane: (block 2 ks: lo, hi), (block 2 ks + 1: lo, hi)
    struct Hdr { uint4v dd; };         // the row's 8 f16 block scales
    struct Consts { half2v s[8]; };
    struct Addr { uint32_t q, h; };
    __device__ static Addr addr(uint32_t tile, int r16, int g32) {
        return Addr{tile + 16u * (uint32_t)(r16 + 32 * g32), tile + (uint32_t)F::kD + 16u * (uint32_t)r16};
    }
    template <int KS, int OFF> __device__ static void read_stage(Stage &st, const Addr &a, uint32_t ring) {
        lds_read128<OFF + KS * 1024>(st.a, a.q + ring);
        lds_read128<OFF + KS * 1024 + 256>(st.b, a.q + ring);
    }
    template <int OFF> __device__ static void read_hdr(Hdr &h, const Addr &a, uint32_t ring) { lds_read128<OFF>(h.dd, a.h + ring); }
    __device__ static void pin_stage(Stage &st) { pin(st.a); pin(st.b); }
    __device__ static void pin_hdr(Hdr &h) { pin(h.dd); }
    __device__ static Consts consts(const Hdr &h, int, _Float16 ws) {
        const uint32_t dw[4] = {h.dd.x, h.dd.y, h.dd.z, h.dd.w};
        Consts c;
#pragma unroll
        for (int i = 0; i < 8; i++) c.s[i] = splat2(h_from_bits((i & 1) ? dw[i >> 1] >> 16 : dw[i >> 1] & 0xFFFFu) * ws);
        return c;
    }
    __device__ static half8v bmin(const Consts &) { return half8v{}; }
    template <int KS, int ST> __device__ static half8v operand(const Stage &st, const Consts &c) {
        constexpr int blk = 2 * KS + (ST >> 1);
        const uint4v src = (ST & 1) ? st.b : st.a;
        const uint32_t w0 = (ST >> 1) ? src.z : src.x, w1 = (ST >> 1) ? src.w : src.y;
        const half2v k1152 = splat2((_Float16)1152.0f);
        return make_half8((and_or_asm_h2(w0, 0x00FF00FFu, kMagic1024) - k1152) * c.s[blk],
                          (and_or_asm_h2(w0 >> 8, 0x00FF00FFu, kMagic1024) - k1152) * c.s[blk],
                          (and_or_asm_h2(w1, 0x00FF00FFu, kMagic1024) - k1152) * c.s[blk],
                          (and_or_asm_h2(w1 >> 8, 0x00FF00FFu, kMagic1024) - k1152) * c.s[blk]);
    }
};

// frags: 32-row fragments, 1 KiB block index (mt * ntc + b) * 17 + q
// vec_out: rows of y can be written as aligned 16-byte pieces
// SK: the columns (k) of every workgroup tile are split over `split` workgroups (split divides the number of super-blocks).
// Each of them - wave by wave, a wave meets only the same wave of the others - writes its partial accumulators to `partials`
// and counts itself in on the tile's counter; the wave that finds all the others counted adds the partial tiles up in part
// order, stores the results and puts the counter back to zero for the next launch.  Nobody waits
// for anybody, and the sums of a result are the same numbers in the same order on every run.  The partial tiles are written
// and read with the cache policy of device-scope atomics (the L2 caches of the XCDs are not coherent with each other), each
// wave's stores have completed before its increment goes out and the last wave reads only after its own has returned.
//   partials: [tile][part][wave] blocks of WM * WN KiB x 4 (a wave's accumulators as its lanes hold them), counters: [tile][wave],
//   zero before the first launch; launches that share them must not overlap.
// KG = 2 (low tile): eight waves as two groups of four.  Group g walks the super-blocks g, g + 2, ... of the workgroup's share
// through rings of its own with the copy schedule, the waits and the barriers of the four-wave form (all eight waves pass the
// same barriers, so the share must be an even number of super-blocks), which puts two waves on every SIMD; after the loop the
// second group hands its accumulators to the first through the LDS.
template <int DT, int WGM_, bool SK = false, int KG = 1>
__global__ void __launch_bounds__(256 * KG) gemm_kq_kernel(GemmGroup grp, int64_t k, const uint8_t *__restrict__ frags, int64_t m, int yt,
                                                           int nblocks_n, int nblocks_m, int vec_out, int split = 1,
                                                           uint8_t *__restrict__ partials = nullptr, uint32_t partial_bytes = 0,
                                                           uint32_t *__restrict__ counters = nullptr) {
    using Fm = GFmt<DT>;
    using G = Geo<DT, WGM_>;
    constexpr int WGN = G::WGN, WM = G::WM, WN = G::WN, TB = G::TB;
    constexpr bool SUMS = Fm::SUMS;
    // Workgroups of one XCD (blockIdx % 8) get consecutive logical ids and the m-blocks of one n-block are
    // consecutive in that order: the packed weights they share stay in that XCD's L2.
    const int nwg = nblocks_n * nblocks_m * (SK ? split : 1);
    int lid = blockIdx.x;
    if ((nwg & 7) == 0) lid = (blockIdx.x & 7) * (nwg >> 3) + (blockIdx.x >> 3);
    // (split: the m-blocks of one n-block and one part are consecutive, they share the part's packed weights)
    int mb = lid % nblocks_m, nb_all = lid / (nblocks_m * (SK ? split : 1));
    const int part = SK ? (lid / nblocks_m) % split : 0;
    if constexpr (!SK) {
        // Many m-blocks (prompts of 1024 rows and more): the workgroups that run together on an XCD - consecutive logical ids -
        // should share activation fragments as well as weights.  With the m-blocks of an n-block all next to each other, 32
        // neighbours are 2 n-blocks x 16 m-blocks: every m-block's fragments (1.1 MB) are then fetched into the L2 once per PAIR of
        // n-blocks (measured at m = 2048, n = 12288: 456 MB fetched per launch for 46 MB of weights and fragments).  In chunks of
        // kChunk m-blocks, 32 neighbours are 8 n-blocks x 4 m-blocks (Q4_K 12288 x 4096: 210 -> 205 us at m = 2048, 421 -> 402 us
        // at m = 4096, same session).
        constexpr int kChunk = 4;
        if (nblocks_m > kChunk) {
            const int per_chunk = kChunk * nblocks_n, chunk = lid / per_chunk, rem = lid - chunk * per_chunk;
            const int left = nblocks_m - chunk * kChunk, mc = left < kChunk ? left : kChunk;
            nb_all = rem / mc;
            mb = chunk * kChunk + rem - nb_all * mc;
        }
    }
    // the weight this n-block belongs to
    const uint8_t *__restrict__ w = grp.w[0];
    void *__restrict__ y = grp.y[0];
    const float *__restrict__ bias = grp.bias[0];
    int64_t n = grp.n[0], ldy = grp.ldy[0];
    float wscale = grp.wscale[0];
    int nb = nb_all;
#pragma unroll
    for (int i = 1; i < kMaxGroup; i++)
        if (i < grp.count && nb_all >= grp.first[i]) {
            w = grp.w[i];
            y = grp.y[i];
            bias = grp.bias[i];
            n = grp.n[i];
            ldy = grp.ldy[i];
            wscale = grp.wscale[i];
            nb = nb_all - grp.first[i];
        }
    // every block scale is multiplied by wscale (a power of two chosen per tensor so that the largest packed-f16 weight
    // lands near 2^15) and the results by its inverse: small scales keep their precision instead of dropping into the
    // f16 subnormals (d * sc / 16 of Q5_K does so from d around 1e-4)
    const _Float16 ws = (_Float16)wscale;
    const float inv_ws = 1.0f / wscale;  // (a power of two: exact)
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    static_assert(KG == 1 || (KG == 2 && G::LOW), "two groups of waves: the low tile only");
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = KG > 1 ? wave_all >> 2 : 0;             // the wave's group and its place in it
    const int wave = KG > 1 ? (wave_all & 3) : wave_all;
    const int wm = wave / WGN, wn = wave % WGN;
    const int n32 = lane & 31, g32 = lane >> 5;
    const int r16 = n32 & 15, tsel = n32 >> 4;
    const int ntc = (int)turq_tile_cols(k);         // super-blocks of a row: the strides of the weights and of the fragments
    const int nloc = (SK ? ntc / split : ntc) / KG;  // ... of this group of waves: kb0, kb0 + KG, ... (nloc of them)
    const int kb0 = part * nloc * KG + kg;
    const int64_t mtiles = (m + 31) / 32;
    const int nrt = (int)turq_tile_rows(n);
    constexpr uint32_t GROUP_BYTES = (uint32_t)(G::S_OFF + (SUMS ? NS * S_BYTES : 0) + 1023) & ~1023u;  // rings of one group of waves
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds + (uint32_t)kg * GROUP_BYTES;
    const uint32_t lane_off = 16u * (uint32_t)lane;

    // ---- copy schedule (all wave-uniform except the per-lane weight offsets) ----
    // activations: this wave's m-tile; one past the end re-reads the last valid tile (never stored)
    // (low form: two waves per m-tile, two of its four steps each; sums block of m-tile wave % 2 into slot `wave`)
    int64_t my_mt = (int64_t)mb * G::GMT + (G::LOW ? wave >> 1 : wave);
    my_mt = my_mt < mtiles ? my_mt : mtiles - 1;
    int64_t my_mt_s = G::LOW ? (int64_t)mb * G::GMT + (wave & 1) : my_mt;
    my_mt_s = my_mt_s < mtiles ? my_mt_s : mtiles - 1;
    const uint32_t a_half = G::LOW ? (uint32_t)(wave & 1) * 2048u : 0u;
    const uint8_t *a_src = uniform_ptr(frags + ((size_t)((my_mt * ntc + kb0) * 17) << 10) + a_half);
    const uint8_t *s_src = uniform_ptr(frags + ((size_t)((my_mt_s * ntc + kb0) * 17) << 10));
    const uint32_t a_dst = lds_base + G::A_OFF + (uint32_t)(G::LOW ? wave >> 1 : wave) * 4096u + a_half;  // + ks * A_STAGE (+ step * 1024)
    const uint32_t s_dst = lds_base + G::S_OFF + (uint32_t)wave * 1024u;  // + (b & 1) * S_BYTES
    // weights: copy c of a super-block covers bytes [1024 c, 1024 c + 1024) of the concatenated tiles of the workgroup;
    // group g = 0..3 holds copies 4g + wave and 16 + 4g + wave (clamped to the last copy; lanes past the end of the
    // tiles re-read the last 16 bytes into the padding of the ring entry)
    const int tile0 = nb * G::NT16;
    const uint8_t *w_src = uniform_ptr(w + ((size_t)tile0 * ntc + kb0) * TB);  // + b * TB
    // (wide form: copies wave, wave + 4, ... of the super-block, CPW per wave, in two halves)
    constexpr int NG = G::WIDE ? G::CPW : 4, NI = G::WIDE ? 1 : 2;
    uint32_t w_voff[NG][NI];
    uint32_t w_dst[NG][NI];
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int i = 0; i < NI; i++) {
            int c = G::WIDE ? 4 * g + wave : (i == 0 ? 4 * g + wave : 16 + 4 * g + wave);
            c = c < G::W_CHUNKS ? c : G::W_CHUNKS - 1;
            uint32_t o = (uint32_t)c * 1024u + lane_off;
            o = o < (uint32_t)G::W_BYTES ? o : (uint32_t)G::W_BYTES - 16u;
            const uint32_t t = o / (uint32_t)TB;
            const uint32_t within = o - t * (uint32_t)TB;
            int tg = tile0 + (int)t;
            tg = tg < nrt ? tg : nrt - 1;  // row tiles past the end re-read the last one (never stored)
            w_voff[g][i] = (uint32_t)(tg - tile0) * (uint32_t)ntc * (uint32_t)TB + within;
            w_dst[g][i] = lds_base + G::W_OFF + (uint32_t)c * 1024u;  // + ring offset
        }
    // ring offsets of the weight buffers of super-blocks b, b + 1, b + 2
    uint32_t wr0 = 0, wr1 = G::W_STRIDE, wr2 = 2 * G::W_STRIDE;

    auto issue_a = [&](int bb, int ks) {  // stage (bb, ks) -> stage buffer ks (wide form: ks % 2)
        const uint8_t *src = a_src + ((size_t)(bb * (KG * 17) + 4 * ks) << 10);
        dma_set<0>(lane_off, src, a_dst + (uint32_t)(ks % G::RA) * G::GA_STAGE);
        dma_more<1024>(lane_off, src);
        if constexpr (!G::LOW) {
            dma_more<2048>(lane_off, src);
            dma_more<3072>(lane_off, src);
        }
    };
    auto issue_w = [&](int bb, int g, uint32_t ring) {  // group g of super-block bb
        const uint8_t *src = w_src + (size_t)bb * (KG * TB);
        if constexpr (G::WIDE) {  // half g of the wave's copies
#pragma unroll
            for (int i = 0; i < G::CPW / 2; i++) dma_set<0>(w_voff[g * (G::CPW / 2) + i][0], src, w_dst[g * (G::CPW / 2) + i][0] + ring);
        } else {
            dma_set<0>(w_voff[g][0], src, w_dst[g][0] + ring);
            dma_set<0>(w_voff[g][1], src, w_dst[g][1] + ring);
        }
    };
    auto issue_s = [&](int bb) {
        if constexpr (SUMS) dma_set<0>(lane_off, s_src + ((size_t)(bb * (KG * 17) + 16) << 10), s_dst + (uint32_t)(bb & 1) * S_BYTES);
    };

    // ---- LDS read addresses ----
    // activations: stage ks, m-tile 2 wm + i, step st at A_OFF + ks * A_STAGE + ((2 wm + i) * 4 + st) * 1024
    const uint32_t a_rd = lds_base + G::A_OFF + (uint32_t)wm * (WM * 4096u) + lane_off;
    const uint32_t s_rd = lds_base + G::S_OFF + (uint32_t)wm * (WM * 1024u) + lane_off;
    // weights: 32-row tile j of this wave = 16-row tiles 2 WN wn + 2 j + tsel of the ring entry
    const typename Fm::Addr w_rd = Fm::addr(lds_base + G::W_OFF + (uint32_t)(2 * WN * wn + tsel) * TB, r16, g32);

    float16v acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // ---- prologue: super-block 0 complete, weights of 1 and the first group of 2 on their way ----
    const int last = nloc - 1;
    if constexpr (G::WIDE) {
        // stages 0 and 1 and the weights of super-block 0 complete, the first half of super-block 1 on its way
        issue_a(0, 0);
        issue_a(0, 1);
        issue_w(0, 0, wr0);
        issue_w(0, 1, wr0);
        issue_w(1 < last ? 1 : last, 0, wr1);
        issue_s(0);
    } else {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) issue_a(0, ks);
#pragma unroll
        for (int g = 0; g < 4; g++) issue_w(0, g, wr0);
#pragma unroll
        for (int g = 0; g < 4; g++) issue_w(1 < last ? 1 : last, g, wr1);
        issue_w(2 < last ? 2 : last, 0, wr2);
        issue_s(0);
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    half8v af[2][WM];  // [step parity][m-tile]
    half8v sf[WM];
    typename Fm::Stage wq[2][WN];  // [stage parity][n-tile]: the packed weights of the stage
    typename Fm::Hdr hd[WN];
    typename Fm::Consts cs[WN], cs_next[WN];
    static_for<WN>([&](auto J) {
        constexpr int j = decltype(J)::value;
        Fm::template read_hdr<j * 2 * TB>(hd[j], w_rd, wr0);
        Fm::template read_stage<0, j * 2 * TB>(wq[0][j], w_rd, wr0);
    });
    static_for<WM>([&](auto I) { lds_read128<decltype(I)::value * 4096>(af[0][decltype(I)::value], a_rd); });
    wait_lds<0>();
#pragma unroll
    for (int j = 0; j < WN; j++) {
        Fm::pin_hdr(hd[j]);
        cs[j] = Fm::consts(hd[j], g32, ws);
    }

    for (int b = 0; b < nloc; b++) {
        const uint32_t s_cur = s_rd + (uint32_t)(b & 1) * S_BYTES;
        const int b1 = b + 1 < last ? b + 1 : last, b2 = b + 2 < last ? b + 2 : last, b3 = b + 3 < last ? b + 3 : last;
        static_for<4>([&](auto KS) {  // the four stages of the super-block: ks selects registers, buffers and offsets
            constexpr int ks = decltype(KS)::value;
            constexpr int cur = ks & 1, nxt = cur ^ 1;
            // entering: wq[cur], af[0] (step 0) and, for ks == 3, hd are in flight
            static_for<4>([&](auto ST) {
                constexpr int st = decltype(ST)::value;
                constexpr int pa = st & 1;
                if constexpr (st < 3) {
                    // next step's activation fragments come in while this step computes
                    static_for<WM>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        lds_read128<(ks % G::RA) * G::GA_STAGE + i * 4096 + (st + 1) * 1024>(af[pa ^ 1][i], a_rd);
                    });
                    wait_lds<WM>();  // everything but the reads just issued
#pragma unroll
                    for (int i = 0; i < WM; i++) pin(af[pa][i]);
                    if constexpr (st == 0) {
#pragma unroll
                        for (int j = 0; j < WN; j++) Fm::pin_stage(wq[cur][j]);
                        if constexpr (ks == 3) {
#pragma unroll
                            for (int j = 0; j < WN; j++) {
                                Fm::pin_hdr(hd[j]);
                                cs_next[j] = Fm::consts(hd[j], g32, ws);
                            }
                        }
                    }
                } else {
                    // ---- stage boundary, before the last step: the next stage becomes readable ----
                    wait_lds<0>();  // step 3's fragments are in registers: this wave is done with the stage's LDS
#pragma unroll
                    for (int i = 0; i < WM; i++) pin(af[1][i]);
                    // The next stage's copies were issued three boundaries ago; younger than them are that
                    // boundary's weight (and sums) copies and everything of the two boundaries since.
                    if constexpr (G::WIDE) {
                        // The next stage's copies were issued at the previous boundary, first of what was issued there; the
                        // boundaries (b, 3) and (b, 0) add half a super-block of weights after them, (b, 1) the sums.  The
                        // waits at (b, 2) and (b, 3) leave nothing in flight, which also completes super-block b + 1 before
                        // its header is read.
                        if constexpr (ks == 0 || ks == 1) wait_vmcnt<G::CPW / 2>(); else wait_vmcnt<0>();
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                        // stage buffer ks % 2 is free: the stage after the next goes there
                        if constexpr (ks < 2) issue_a(b, ks + 2); else issue_a(b1, ks - 2);
                        if constexpr (ks == 0) issue_w(b1, 1, wr1);       // second half of super-block b + 1
                        if constexpr (ks == 3) issue_w(b2, 0, wr0);       // first half of super-block b + 2: b's buffer is free
                        if constexpr (ks == 1) issue_s(b1);
                    } else {
                    if constexpr (ks == 0 || !SUMS) wait_vmcnt<14>(); else wait_vmcnt<15>();
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    // now stage buffer ks is free: stage (b + 1, ks) goes there
                    issue_a(b1, ks);
                    if constexpr (ks == 3) issue_w(b3, 0, wr0); else issue_w(b2, ks + 1, wr2);
                    if constexpr (ks == 0) issue_s(b1);
                    }
                    // first reads of the next stage, hidden under step 3's MFMAs
                    if constexpr (ks == 3 && SUMS) {
                        static_for<WM>([&](auto I) { lds_read128<decltype(I)::value * 1024>(sf[decltype(I)::value], s_cur); });
                    }
                    constexpr int nks = (ks + 1) & 3;
                    const uint32_t ring_from = ks == 3 ? wr1 : wr0;
                    static_for<WN>([&](auto J) {
                        constexpr int j = decltype(J)::value;
                        Fm::template read_stage<nks, j * 2 * TB>(wq[nxt][j], w_rd, ring_from);
                    });
                    if constexpr (ks == 2) {
                        static_for<WN>([&](auto J) {
                            constexpr int j = decltype(J)::value;
                            Fm::template read_hdr<j * 2 * TB>(hd[j], w_rd, wr1);
                        });
                    }
                    static_for<WM>([&](auto I) { lds_read128<(nks % G::RA) * G::GA_STAGE + decltype(I)::value * 4096>(af[0][decltype(I)::value], a_rd); });
                }
                // operand step 4 ks + st of the lane's 128 columns
                half8v bop[WN];
#pragma unroll
                for (int j = 0; j < WN; j++) bop[j] = Fm::template operand<ks, st>(wq[cur][j], cs[j]);
#pragma unroll
                for (int i = 0; i < WM; i++)
#pragma unroll
                    for (int j = 0; j < WN; j++) acc[i][j] = mfma32x32x16(af[pa][i], bop[j], acc[i][j]);
            });
            if constexpr (ks == 3) {
                if constexpr (SUMS) {
                    // "- dmin * m" term against the sub-block sums
                    wait_lds<WN * Fm::NSTG + WM>();  // all but the weight and fragment reads of the next stage
#pragma unroll
                    for (int i = 0; i < WM; i++) pin(sf[i]);
#pragma unroll
                    for (int i = 0; i < WM; i++)
#pragma unroll
                        for (int j = 0; j < WN; j++) acc[i][j] = mfma32x32x16(sf[i], Fm::bmin(cs[j]), acc[i][j]);
                }
                // the next super-block's constants take over
#pragma unroll
                for (int j = 0; j < WN; j++) cs[j] = cs_next[j];
            }
        });
        const uint32_t t = wr0;
        wr0 = wr1;
        if constexpr (G::WIDE) {
            wr1 = t;
        } else {
            wr1 = wr2;
            wr2 = t;
        }
    }
    wait_lds<0>();
    // The last stage boundary has issued the first LDS reads of a stage that does not exist.  Nothing uses them, but they
    // are asm statements: the compiler takes their destination registers for written when the statement executes and, the
    // values being dead, hands the registers out again at once, while the data arrives whenever the LDS delivers it.  (A
    // division placed here by the compiler lost its temporaries that way, in whole wave tiles of some launches.)  Naming
    // the registers after the wait keeps them reserved until the reads have landed.
#pragma unroll
    for (int i = 0; i < WM; i++) pin(af[0][i]);
#pragma unroll
    for (int j = 0; j < WN; j++) Fm::pin_stage(wq[0][j]);
    wait_vmcnt<0>();  // the trailing copies must neither outlive the workgroup's LDS nor land in the staged results
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    if constexpr (KG > 1) {
        // ---- the second group of waves hands its sums to the first (behind the staged results' part of the LDS) ----
        constexpr int NQ = WM * WN * 4;
        float4v *red = (float4v *)(lds + 4 * WM * 32 * G::OUT_PITCH * 4) + (size_t)wave * (NQ * 64) + lane;
        if (kg == 1) {
#pragma unroll
            for (int i = 0; i < WM; i++)
#pragma unroll
                for (int j = 0; j < WN; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        red[((i * WN + j) * 4 + q) * 64] = float4v{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int i = 0; i < WM; i++)
#pragma unroll
            for (int j = 0; j < WN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4v f = red[((i * WN + j) * 4 + q) * 64];
                    acc[i][j][4 * q] += f.x;
                    acc[i][j][4 * q + 1] += f.y;
                    acc[i][j][4 * q + 2] += f.z;
                    acc[i][j][4 * q + 3] += f.w;
                }
    }

    if constexpr (SK) {
        // ---- the parts of a tile meet (no workgroup barrier from here on: a wave may leave alone) ----
        constexpr int NB = WM * WN * 4;                 // 1 KiB blocks of a wave's partial tile (16 bytes per lane each)
        constexpr uint32_t WAVE_BYTES = NB * 1024u;
        constexpr int PB = NB >= 32 ? 1 : 32 / NB;      // parts read together: 128 registers of loads in flight per lane
        const int tile = nb_all * nblocks_m + mb;
        uint32_t *cnt = counters + tile * 4 + wave;
        const __amdgpu_buffer_rsrc_t prs = __builtin_amdgcn_make_buffer_rsrc(partials, 0, (int)partial_bytes, 0x00020000);
        const uint32_t tile_base = (uint32_t)(tile * split) * (4u * WAVE_BYTES) + (uint32_t)wave * WAVE_BYTES + lane_off;
        const uint32_t mine = tile_base + (uint32_t)part * (4u * WAVE_BYTES);
#pragma unroll
        for (int i = 0; i < WM; i++)
#pragma unroll
            for (int j = 0; j < WN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4v v = float4v{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, v), prs, mine + (uint32_t)((i * WN + j) * 4 + q) * 1024u, 0,
                                                           kCoherent);
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        uint32_t ticket = 0;
        if (lane == 0) ticket = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (__builtin_amdgcn_readfirstlane(ticket) != (uint32_t)(split - 1)) return;
        // the last one in: every part's tile, its own from its registers, added in part order
        float16v sum[WM][WN];
#pragma unroll
        for (int i = 0; i < WM; i++)
#pragma unroll
            for (int j = 0; j < WN; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) sum[i][j][e] = 0.0f;
        for (int p0 = 0; p0 < split; p0 += PB) {
            if (PB == 1 && p0 == part) {
#pragma unroll
                for (int i = 0; i < WM; i++)
#pragma unroll
                    for (int j = 0; j < WN; j++) sum[i][j] += acc[i][j];
                continue;
            }
            // (several parts at once: the wave's own among them, as it has just written it; parts past the last: the last
            // one again, not added)
            uint4v v[PB][NB];
#pragma unroll
            for (int b = 0; b < PB; b++) {
                const uint32_t from = tile_base + (uint32_t)(p0 + b < split ? p0 + b : split - 1) * (4u * WAVE_BYTES);
#pragma unroll
                for (int t = 0; t < NB; t++) v[b][t] = __builtin_amdgcn_raw_buffer_load_b128(prs, from + (uint32_t)t * 1024u, 0, kCoherent);
            }
#pragma unroll
            for (int b = 0; b < PB; b++) {
                if (p0 + b >= split) break;
#pragma unroll
                for (int i = 0; i < WM; i++)
#pragma unroll
                    for (int j = 0; j < WN; j++)
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const float4v f = __builtin_bit_cast(float4v, v[b][(i * WN + j) * 4 + q]);
                            sum[i][j][4 * q] += f.x;
                            sum[i][j][4 * q + 1] += f.y;
                            sum[i][j][4 * q + 2] += f.z;
                            sum[i][j][4 * q + 3] += f.w;
                        }
            }
        }
#pragma unroll
        for (int i = 0; i < WM; i++)
#pragma unroll
            for (int j = 0; j < WN; j++) acc[i][j] = sum[i][j];
        if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- results ----
    // 32x32 result: lane (n32, g32), register e holds row 8 * (e / 4) + 4 * g32 + e % 4 of column n32
    constexpr int OUT_PITCH = G::OUT_PITCH;
    const bool accum = (yt & TURQ_OUT_ACCUMULATE) != 0;  // y += results: the residual stream
    const int ytb = yt & 0xFF;
    const int64_t row0 = (int64_t)mb * G::GBM + wm * (WM * 32);
    const int64_t col0 = (int64_t)nb * G::BN + wn * (WN * 32);
    if (vec_out) {
        float *stage = (float *)lds + (size_t)wave * (WM * 32 * OUT_PITCH);
#pragma unroll
        for (int j = 0; j < WN; j++) {
            const int64_t col = col0 + 32 * j + n32;
            const float bv = (bias && col < n) ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < WM; i++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                    stage[(32 * i + 8 * (e >> 2) + 4 * g32 + (e & 3)) * OUT_PITCH + 32 * j + n32] = acc[i][j][e] * inv_ws + bv;
        }
        // each wave reads back only what it wrote itself; LDS operations of one wave complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        uint64_t badm = 0;  // results that are no finite numbers, or do not fit an f16 output (turq_ctx_nonfinite_count)
        const float lim = turq_finite_limit(ytb);
        if (ytb == TURQ_ACT_F32) {
            constexpr int CPR = WN * 32 / 4;  // 16-byte pieces per row
#pragma unroll 4
            for (int it = 0; it < WM * 32 * CPR / 64; it++) {
                const int c = it * 64 + lane;
                const int r = c / CPR, cc = c - r * CPR;
                float4v v = *(const float4v *)(stage + r * OUT_PITCH + 4 * cc);
                if (row0 + r < m && col0 + 4 * cc < n) {
                    float4v *dst = (float4v *)((float *)y + (row0 + r) * ldy + col0 + 4 * cc);
                    if (accum) v += *dst;
                    badm |= note_mask(v.x, lim) | note_mask(v.y, lim) | note_mask(v.z, lim) | note_mask(v.w, lim);
                    __builtin_nontemporal_store(v, dst);
                }
            }
        } else {
            constexpr int CPR = WN * 32 / 8;
#pragma unroll 4
            for (int it = 0; it < WM * 32 * CPR / 64; it++) {
                const int c = it * 64 + lane;
                const int r = c / CPR, cc = c - r * CPR;
                const float4v v0 = *(const float4v *)(stage + r * OUT_PITCH + 8 * cc);
                const float4v v1 = *(const float4v *)(stage + r * OUT_PITCH + 8 * cc + 4);
                if (row0 + r < m && col0 + 8 * cc < n) {
                    uint4v *dst = (uint4v *)((uint16_t *)y + (row0 + r) * ldy + col0 + 8 * cc);
                    float vs[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                    if (accum) {
                        const uint4v old = *dst;
                        const uint32_t ow[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            if (ytb == TURQ_ACT_BF16) {
                                vs[2 * e] += __uint_as_float(ow[e] << 16);
                                vs[2 * e + 1] += __uint_as_float(ow[e] & 0xFFFF0000u);
                            } else {
                                const half2v hh = as_half2(ow[e]);
                                vs[2 * e] += (float)hh.x;
                                vs[2 * e + 1] += (float)hh.y;
                            }
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 8; e++) badm |= note_mask(vs[e], lim);
                    uint4v o;
                    if (ytb == TURQ_ACT_BF16)
                        o = uint4v{pack_bf16x2(vs[0], vs[1]), pack_bf16x2(vs[2], vs[3]), pack_bf16x2(vs[4], vs[5]), pack_bf16x2(vs[6], vs[7])};
                    else
                        o = uint4v{pack_f16x2(vs[0], vs[1]), pack_f16x2(vs[2], vs[3]), pack_f16x2(vs[4], vs[5]), pack_f16x2(vs[6], vs[7])};
                    __builtin_nontemporal_store(o, dst);
                }
            }
        }
        turq_note_flush(badm != 0 ? 1u : 0u);
    } else {
        uint64_t badm = 0;
        const float lim = turq_finite_limit(ytb);
#pragma unroll
        for (int j = 0; j < WN; j++) {
            const int64_t col = col0 + 32 * j + n32;
            if (col >= n) continue;
            const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < WM; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int64_t row = row0 + 32 * i + 8 * (e >> 2) + 4 * g32 + (e & 3);
                    if (row < m) {
                        float v = acc[i][j][e] * inv_ws + bv;
                        if (accum)
                            v += ytb == TURQ_ACT_F32 ? turq_load_out<TURQ_ACT_F32>(y, row * ldy + col)
                                 : ytb == TURQ_ACT_BF16 ? turq_load_out<TURQ_ACT_BF16>(y, row * ldy + col) : turq_load_out<TURQ_ACT_F16>(y, row * ldy + col);
                        badm |= note_mask(v, lim);
                        if (ytb == TURQ_ACT_F32) turq_store_out_raw<TURQ_ACT_F32>(y, row * ldy + col, v);
                        else if (ytb == TURQ_ACT_BF16) turq_store_out_raw<TURQ_ACT_BF16>(y, row * ldy + col, v);
                        else turq_store_out_raw<TURQ_ACT_F16>(y, row * ldy + col, v);
                    }
                }
        }
        turq_note_flush(badm != 0 ? 1u : 0u);
    }
}

// split > 1: the columns of every tile over `split` workgroups that meet in `partials`, counted on `counters`
// (kSplitCounterBytes, zero between launches)
constexpr size_t kSplitCounterBytes = TURQ_GEMM_SPLIT_COUNTER_BYTES;
template <int DT, int WGM_, bool SK = false, int KG = 1>
hipError_t launch_gemm(const TurqGemmWeights &ws, int64_t k, const void *frags, int64_t m, int y_dtype, hipStream_t stream,
                       hipEvent_t ev_start, hipEvent_t ev_stop, int split = 1, void *counters = nullptr, void *partials = nullptr,
                       size_t partials_cap = 0) {
    using G = Geo<DT, WGM_>;
    constexpr int RING_BYTES = KG * ((G::S_OFF + (GFmt<DT>::SUMS ? NS * S_BYTES : 0) + 1023) & ~1023);
    // (after the main loop: the staged results, behind them the sums that a second group of waves hands over)
    constexpr int STAGING_BYTES = 4 * G::WM * 32 * G::OUT_PITCH * 4 + (KG > 1 ? 4 * G::WM * G::WN * 4096 : 0);
    constexpr int LDS_BYTES = RING_BYTES > STAGING_BYTES ? RING_BYTES : STAGING_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of one workgroup: the rings, or the staged results after the main loop");
    // per-lane weight offsets are 32-bit
    if ((uint64_t)G::NT16 * (uint64_t)(k / 256) * G::TB >= (1ull << 32)) return hipErrorInvalidValue;
    if ((k / 256 / (SK ? split : 1)) % KG != 0) return hipErrorInvalidValue;
    if (ws.count < 1 || ws.count > kMaxGroup) return hipErrorInvalidValue;
    const hipError_t attr = turq_raise_lds_limit((const void *)gemm_kq_kernel<DT, WGM_, SK, KG>, LDS_BYTES);
    if (attr != hipSuccess) return attr;
    GemmGroup grp{};
    grp.count = ws.count;
    const int es = (y_dtype & 0xFF) == TURQ_ACT_F32 ? 4 : 2;
    int nbn = 0, vec_out = 1;
    for (int i = 0; i < ws.count; i++) {
        grp.w[i] = (const uint8_t *)ws.w[i];
        grp.y[i] = ws.y[i];
        grp.bias[i] = ws.bias[i];
        grp.n[i] = ws.n[i];
        grp.ldy[i] = ws.ldy[i];
        grp.wscale[i] = ws.wscale[i];
        grp.first[i] = nbn;
        nbn += (int)((ws.n[i] + G::BN - 1) / G::BN);
        // rows of y can be written as aligned 16-byte pieces (every weight of the launch, or none)
        vec_out = vec_out && (uintptr_t)ws.y[i] % 16 == 0 && ((uint64_t)ws.ldy[i] * es) % 16 == 0 && ws.n[i] % 8 == 0;
    }
    const int nbm = (int)((m + G::GBM - 1) / G::GBM);
    size_t partial_bytes = 0;
    if constexpr (SK) {
        partial_bytes = (size_t)nbn * nbm * split * (size_t)(G::WM * G::WN * 4 * 4096);
        if (split < 2 || (k / 256) % split != 0 || !counters || !partials || (size_t)nbn * nbm * 16 > kSplitCounterBytes ||
            partial_bytes >= (1ull << 31) || partial_bytes > partials_cap)
            return hipErrorInvalidValue;
    } else {
        split = 1;
    }
    const dim3 grid((unsigned)(nbn * nbm * split)), block(256 * KG);
    if (ev_start) {
        hipExtLaunchKernelGGL((gemm_kq_kernel<DT, WGM_, SK, KG>), grid, block, LDS_BYTES, stream, ev_start, ev_stop, 0, grp, k,
                              (const uint8_t *)frags, m, y_dtype, nbn, nbm, vec_out, split, (uint8_t *)partials, (uint32_t)partial_bytes,
                              (uint32_t *)counters);
    } else {
        gemm_kq_kernel<DT, WGM_, SK, KG><<<grid, block, LDS_BYTES, stream>>>(grp, k, (const uint8_t *)frags, m, y_dtype, nbn, nbm, vec_out, split,
                                                                          (uint8_t *)partials, (uint32_t)partial_bytes, (uint32_t *)counters);
    }
    return hipGetLastError();
}

}  // namespace

// The workgroup tile of a launch: 1: 128 x 128 (1 x 4 waves), 2: 2 x 2 waves (Q4_K 128 x 192, Q8_0 128 x 64), 3: wide 128 x 256,
// 4: low 64 x 128; 0: no kernel for this format.  compute_units: CUs of the device (0: unknown).
int turq_gemm_form(int dtype, int64_t n, int64_t k, int64_t m, int compute_units) {
    (void)k;
    const bool tall = !turq_tuning().gemm_grid_2x2;  // Q5_K / Q6_K: 1 x 4 waves unless told otherwise
    // The wide tile (128 x 256, Geo<.., 3>) pulls fewer activation bytes through the L2 per flop (Q4_K: + 12 % at m = 2048 and
    // 4096; LM head Q5_K / Q6_K: + 4 .. 21 % from m = 64 to 512) but makes fewer, larger workgroups: it is taken where its
    // gain outweighs what its workgroup count loses in the last round over the CUs, and only where there are workgroups
    // enough to matter.  TURQ_GEMM_WIDE = 0 / 1 overrides the rule.
    const int wide_env = turq_tuning().gemm_wide;
    const int64_t cus = compute_units > 0 ? compute_units : 256;
    auto fill = [&](int64_t bn, int64_t *count) {  // share of the CU-rounds a launch with this tile width keeps busy
        const int64_t wgs = ((n + bn - 1) / bn) * ((m + BM - 1) / BM), rounds = (wgs + cus - 1) / cus;
        if (count) *count = wgs;
        return (double)wgs / (double)(rounds * cus);
    };
    int64_t wide_wgs = 0;
    const double fill_wide = fill(256, &wide_wgs);
    auto pick_wide = [&](int64_t bn_other, double gain) {
        if (wide_env >= 0) return wide_env == 1;
        return 2 * wide_wgs >= cus && fill_wide * gain >= fill(bn_other, nullptr);
    };
    // The low tile (64 x 128, Geo<.., 4>) for launches of up to 64 rows, and for those whose 128 x 128 tiles would leave at
    // least half of the CUs without a workgroup (twice the workgroups).  TURQ_GEMM_LOW = 0 / 1 overrides the rule.
    const int low_env = turq_tuning().gemm_low;
    const int64_t wgs128 = ((n + 127) / 128) * ((m + BM - 1) / BM);
    // (up to 64 rows the low tile is the whole problem's height: half the MFMA work and activation traffic of a 128-row tile)
    const bool low = low_env >= 0 ? low_env == 1 : (m <= 64 || 2 * wgs128 <= cus);
    const bool kq = dtype == TURQ_Q4_K || dtype == TURQ_Q5_K || dtype == TURQ_Q6_K;
    if (low && wide_env != 1 && kq) return 4;
    switch (dtype) {
    case TURQ_Q4_K:
        if (wide_env == 1) return 3;
        // 128 x 192 tiles of 2 x 2 waves, unless the 128 x 128 tiles of the 1 x 4 grid still fit the machine in one round:
        // then there are half as many again to spread (m = 128: 96 workgroups instead of 64, 34 us instead of 45)
        if (compute_units > 0 && wgs128 <= compute_units) return 1;
        return pick_wide(192, 1.10) ? 3 : 2;
    case TURQ_Q5_K:
    case TURQ_Q6_K: return pick_wide(128, 1.25) ? 3 : tall ? 1 : 2;
    case TURQ_Q8_0: return 2;
    default: return 0;
    }
}

// ---- which launches split their columns ----
// A launch whose tiles leave most CUs idle - the tall-k matrices of a model at prefill chunk sizes (down_proj 4096 x 12288 makes
// 32 low tiles at 64 rows, 64 wide ones at 512), and every matrix of the layer at 64 rows - gives every tile to `split`
// workgroups.  What the parts' meeting costs grows with the partial tiles the launch writes and reads back (m x n x 4 bytes
// x (2 split - 1)), so the rule takes the low tile for few rows and the wide one above, and only as many parts as leave a
// quarter of the CUs free (low tiles; a quarter of the CUs taken when k is short, and then only up to 128 rows: since the
// low tile runs eight waves there is less to win) or fill them once (wide tiles, up to an eighth of the CUs).  Measured on MI355X, Q6_K 4096 x 12288, no split -> split: 64 rows 75 -> 35 us
// (low, 6 parts), 128: 78 -> 47 (low, 3), 256: 82 -> 66 (wide, 6), 512: 97 -> 92 (wide, 4: within what a whole layer's step
// varies by, not taken), 1024: none helps; Q4_K 4096 x 4096: 64 rows 28 -> 22 us (low, 4), 128: 28 -> 27 (low, 2), from 256
// rows on none helps; 12288 x 4096: none helps; with the eight-wave low tile since: 4096 x 4096 unsplit 21.8 / 22.3 us at 64 /
// 128 rows against 21.1 / 24.2 in 4 / 2 parts, 1024 x 4096 21.6 / 21.8 against 15.3 / 16.9 in 4 parts.  TURQ_GEMM_SPLIT = 0: never, s > 1: by s wherever s divides (with
// TURQ_GEMM_SPLIT_FORM = 3 / 4: on the wide / low tile).
size_t turq_gemm_split_scratch(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int *form_out, int *split_out) {
    if (form_out) *form_out = 0;
    if (split_out) *split_out = 1;
    const int env = turq_tuning().gemm_split, env_form = turq_tuning().gemm_split_form;
    if (env == 0 || compute_units <= 0 || (dtype != TURQ_Q4_K && dtype != TURQ_Q5_K && dtype != TURQ_Q6_K)) return 0;
    const int64_t cus = compute_units, ntc = k / 256;
    const int64_t low_tiles = ((n + 127) / 128) * ((m + 63) / 64), wide_tiles = ((n + 255) / 256) * ((m + 127) / 128);
    // the most parts that divide the super-blocks, leave each part at least min_sb of them and make at most max_wgs workgroups
    auto parts = [&](int64_t tiles, int64_t max_wgs, int64_t min_sb) {
        int best = 1;
        for (int s = 2; s <= 8; s++)
            if (ntc % s == 0 && ntc / s >= min_sb && tiles * s <= max_wgs) best = s;
        return best;
    };
    int form = 0, split = 1;
    if (env > 1) {
        form = env_form == 3 || env_form == 4 ? env_form : (m <= 128 ? 4 : 3);
        split = ntc % env == 0 ? env : 1;
    } else {
        const bool tall = ntc >= 32;
        split = tall || m <= 128 ? parts(low_tiles, tall ? 3 * cus / 4 : cus / 4, 4) : 1;
        form = 4;
        if (split == 1 && tall && 8 * wide_tiles <= cus) {
            split = parts(wide_tiles, cus, 8);
            form = 3;
        }
    }
    if (split < 2) return 0;
    const int64_t bm = form == 4 ? 64 : 128, bn = form == 4 ? 128 : 256;
    const size_t tiles = (size_t)(form == 4 ? low_tiles : wide_tiles), bytes = tiles * (size_t)split * (size_t)(bm * bn * 4);
    if (tiles * 16 > kSplitCounterBytes || bytes > (256u << 20)) return 0;
    if (form_out) *form_out = form;
    if (split_out) *split_out = split;
    return bytes;
}

// The launch the rules above would make for these rows: its workgroups, and the share of its rounds over the CUs that it keeps
// busy, weighted by the wide tile's measured gain.
double turq_gemm_fill(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int64_t *wgs_out) {
    const int form = turq_gemm_form(dtype, n, k, m, compute_units);
    const int64_t cus = compute_units > 0 ? compute_units : 256;
    const int64_t bm = form == 4 ? 64 : 128;
    const int64_t bn = form == 3 ? 256 : form == 2 ? (dtype == TURQ_Q4_K ? 192 : dtype == TURQ_Q8_0 ? 64 : 128) : 128;
    const int64_t wgs = ((n + bn - 1) / bn) * ((m + bm - 1) / bm), rounds = (wgs + cus - 1) / cus;
    if (wgs_out) *wgs_out = wgs;
    const double gain = form == 3 ? (dtype == TURQ_Q4_K ? 1.10 : 1.25) : 1.0;
    return rounds > 0 ? (double)wgs / (double)(rounds * cus) * gain : 0.0;
}

// whether a low-tile launch whose tiles are split over `split` workgroups each takes the eight-wave form (one such workgroup
// fills a CU's LDS; two of the four-wave form share one)
bool turq_gemm_low_two_groups(int64_t n, int64_t k, int64_t m, int split, int compute_units) {
    const int kgroups = turq_tuning().gemm_kgroups;
    if (split < 1 || (k / 256) % split != 0 || (k / 256 / split) % 2 != 0 || kgroups == 1) return false;
    const int64_t wgs = ((n + 127) / 128) * ((m + 63) / 64) * split;
    return kgroups == 2 || wgs <= (compute_units > 0 ? compute_units : 256);
}

// frags: activations prepared by turq_launch_act_prep32 (in the order of the same dtype) for all m rows
// wscale: a power of two in [2^-14, 2^15] by which the kernel multiplies every block scale; compute_units: CUs of the device
// (0: unknown), for the choice of the tile shape
hipError_t turq_launch_gemm_mfma(int dtype, const void *w, int64_t n, int64_t k, const void *frags, int64_t m, void *y,
                                 int y_dtype, int64_t ldy, const float *bias, float wscale, int compute_units, hipStream_t stream,
                                 hipEvent_t ev_start, hipEvent_t ev_stop, void *split_counters, void *split_partials,
                                 size_t split_partial_bytes) {
    TurqGemmWeights ws{};
    ws.count = 1;
    ws.w[0] = w;
    ws.y[0] = y;
    ws.bias[0] = bias;
    ws.n[0] = n;
    ws.ldy[0] = ldy;
    ws.wscale[0] = wscale;
    return turq_launch_gemm_mfma_group(dtype, ws, k, frags, m, y_dtype, compute_units, stream, ev_start, ev_stop, split_counters,
                                       split_partials, split_partial_bytes);
}

// ... for up to four weights of one format in one launch: the tile, the split and the wave groups are chosen for the rows of all
// of them together (every n a multiple of 256, so that no tile of any form straddles two weights)
hipError_t turq_launch_gemm_mfma_group(int dtype, const TurqGemmWeights &ws, int64_t k, const void *frags, int64_t m, int y_dtype,
                                       int compute_units, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop,
                                       void *split_counters, void *split_partials, size_t split_partial_bytes) {
    if (ws.count < 1 || ws.count > 4) return hipErrorInvalidValue;
    int64_t n = 0;
    for (int i = 0; i < ws.count; i++) {
        if (ws.n[i] <= 0 || (ws.count > 1 && ws.n[i] % 256 != 0)) return ws.n[i] == 0 && ws.count == 1 ? hipSuccess : hipErrorInvalidValue;
        if (!(ws.wscale[i] >= 6.103515625e-5f && ws.wscale[i] <= 32768.0f)) return hipErrorInvalidValue;
        n += ws.n[i];
    }
    if (m == 0) return hipSuccess;
    if (k <= 0 || k % 256 != 0) return hipErrorInvalidValue;
    const int form = turq_gemm_form(dtype, n, k, m, compute_units);
    if (form == 0) return hipErrorInvalidValue;
    // The low tile with two groups of waves where a workgroup's share of the super-blocks is even and the launch is at most one
    // workgroup per CU: the second group then fills SIMD time that nothing else would (Q4_K 4096 x 4096 at 256 / 512 rows
    // 29.4 -> 23.4 / 32.6 -> 26.9 us, 12288 x 4096 at 128 rows 29.9 -> 25.2, 1024 x 4096 at 512 rows 30.4 -> 23.1, Q6_K
    // 4096 x 12288 at 512 rows 105 -> 97); with more workgroups than CUs two four-wave workgroups share a CU anyway and the
    // eight-wave one is slower (LM head at 64 rows 178 -> 196 us).  TURQ_GEMM_KGROUPS = 1: never, 2: wherever the share is even.
    auto two_groups_for = [&](int split) { return turq_gemm_low_two_groups(n, k, m, split, compute_units); };
    if (split_counters && split_partials) {
        int sform = 0, split = 1;
        const size_t need = turq_gemm_split_scratch(dtype, n, k, m, compute_units, &sform, &split);
        if (need != 0 && need <= split_partial_bytes) {
            if (sform == 4 && two_groups_for(split)) {
#define TURQ_GEMM_SK2(DT)                                                                                                               \
    return launch_gemm<DT, 4, true, 2>(ws, k, frags, m, y_dtype, stream, ev_start, ev_stop, split, split_counters, split_partials, \
                                       split_partial_bytes)
                switch (dtype) {
                case TURQ_Q4_K: TURQ_GEMM_SK2(TURQ_Q4_K);
                case TURQ_Q5_K: TURQ_GEMM_SK2(TURQ_Q5_K);
                case TURQ_Q6_K: TURQ_GEMM_SK2(TURQ_Q6_K);
                default: break;
                }
#undef TURQ_GEMM_SK2
            }
#define TURQ_GEMM_SK(DT, F)                                                                                                           \
    return launch_gemm<DT, F, true>(ws, k, frags, m, y_dtype, stream, ev_start, ev_stop, split, split_counters, split_partials, \
                                    split_partial_bytes)
            switch (dtype * 8 + sform) {
            case TURQ_Q4_K * 8 + 3: TURQ_GEMM_SK(TURQ_Q4_K, 3);
            case TURQ_Q4_K * 8 + 4: TURQ_GEMM_SK(TURQ_Q4_K, 4);
            case TURQ_Q5_K * 8 + 3: TURQ_GEMM_SK(TURQ_Q5_K, 3);
            case TURQ_Q5_K * 8 + 4: TURQ_GEMM_SK(TURQ_Q5_K, 4);
            case TURQ_Q6_K * 8 + 3: TURQ_GEMM_SK(TURQ_Q6_K, 3);
            case TURQ_Q6_K * 8 + 4: TURQ_GEMM_SK(TURQ_Q6_K, 4);
            default: break;
            }
#undef TURQ_GEMM_SK
        }
    }
    if (form == 4 && two_groups_for(1)) {
#define TURQ_GEMM_2(DT) return launch_gemm<DT, 4, false, 2>(ws, k, frags, m, y_dtype, stream, ev_start, ev_stop)
        switch (dtype) {
        case TURQ_Q4_K: TURQ_GEMM_2(TURQ_Q4_K);
        case TURQ_Q5_K: TURQ_GEMM_2(TURQ_Q5_K);
        case TURQ_Q6_K: TURQ_GEMM_2(TURQ_Q6_K);
        default: break;
        }
#undef TURQ_GEMM_2
    }
#define TURQ_GEMM(DT, F) return launch_gemm<DT, F>(ws, k, frags, m, y_dtype, stream, ev_start, ev_stop)
    switch (dtype * 8 + form) {
    case TURQ_Q4_K * 8 + 1: TURQ_GEMM(TURQ_Q4_K, 1);
    case TURQ_Q4_K * 8 + 2: TURQ_GEMM(TURQ_Q4_K, 2);
    case TURQ_Q4_K * 8 + 3: TURQ_GEMM(TURQ_Q4_K, 3);
    case TURQ_Q4_K * 8 + 4: TURQ_GEMM(TURQ_Q4_K, 4);
    case TURQ_Q5_K * 8 + 1: TURQ_GEMM(TURQ_Q5_K, 1);
    case TURQ_Q5_K * 8 + 2: TURQ_GEMM(TURQ_Q5_K, 2);
    case TURQ_Q5_K * 8 + 3: TURQ_GEMM(TURQ_Q5_K, 3);
    case TURQ_Q5_K * 8 + 4: TURQ_GEMM(TURQ_Q5_K, 4);
    case TURQ_Q6_K * 8 + 1: TURQ_GEMM(TURQ_Q6_K, 1);
    case TURQ_Q6_K * 8 + 2: TURQ_GEMM(TURQ_Q6_K, 2);
    case TURQ_Q6_K * 8 + 3: TURQ_GEMM(TURQ_Q6_K, 3);
    case TURQ_Q6_K * 8 + 4: TURQ_GEMM(TURQ_Q6_K, 4);
    case TURQ_Q8_0 * 8 + 2: TURQ_GEMM(TURQ_Q8_0, 2);
    default: return hipErrorInvalidValue;
    }
#undef TURQ_GEMM
}

TURQ_NONFINITE_READER(turq_nonfinite_gemm_mfma)
