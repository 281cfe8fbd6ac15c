// Device helpers shared by the MFMA kernels: vector types, the "magic number" integer -> f16
// unpack, and the layout of prepared activations.
//
// Integer -> f16 without a convert instruction.  OR-ing a small unsigned field into the mantissa of
// a fixed f16 exponent gives base + field * ulp exactly:
//   bits 0x6400 | v        = 1024 + v          (v < 1024, ulp 1)
//   bits 0x6400 | (v << 4) = 1024 + 16 * v
//   bits 0x5C00 | (v << 2) = 256 + v           (ulp 1/4)
//   bits 0x4C00 | (v << 6) = 16 + v            (ulp 1/64)
// One v_and_or_b32 therefore turns two fields of a packed dword (one per 16-bit half) into a packed
// f16 pair, and one v_pk_fma_f16 with (scale, -base * scale) removes the base and applies an integer
// block scale at the same time.  All products here are integers below 2048, so every value that
// reaches the MFMA is exact; the only rounding on the weight side is none at all.
//
// Prepared activations ("A fragments").  The kernels use v_mfma_f32_16x16x32_f16 with the
// activations as the A operand (16 rows of m) and the weights as the B operand (16 rows of n), so
// lane (n, g) of the result holds y[m = 4g..4g+3][n].  For every 256-column tile b and MFMA step q
// the activation fragment is stored lane-linear, 16 bytes (8 f16) per (g, r):
//   chunk index = (((mt * ntc + b) * NQ + q) * 4 + g) * mpad + r          (mt = m / 16, r = m % 16)
//   K-quants (NQ = 9): q < 8 holds x[m][256b + 64g + 8q + j];  q = 8 holds, for the four
//     16-element groups of lane group g, the group sums of the f16-rounded activations split in
//     two f16 (hi, lo): slots (hi0, lo0, hi1, lo1, hi2, lo2, hi3, lo3)
//   Q8_0 (NQ = 8): q holds x[m][256b + 32q + 8g + j]
// mpad is the m-tile height rounded up to 1, 2, 4, 8 or 16; rows beyond m are zero.
#pragma once

#include <mutex>
#include <set>
#include <utility>

#include "common.h"

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

#define TURQ_NQ_KQUANT 9
#define TURQ_NQ_Q8_0 8

__host__ __device__ inline int turq_mpad(int64_t rows) {
    return rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : rows <= 8 ? 8 : 16;
}
__host__ __device__ inline int turq_nq(int dt) { return dt == TURQ_Q8_0 ? TURQ_NQ_Q8_0 : TURQ_NQ_KQUANT; }
// bytes of the prepared-activation buffer for m rows against a weight of k columns
__host__ __device__ inline size_t turq_act_prep_bytes(int dt, int64_t m, int64_t k) {
    const int64_t mtiles = (m + 15) / 16;
    const int mpad = mtiles > 1 ? 16 : turq_mpad(m);
    return (size_t)mtiles * (size_t)((k + 255) / 256) * (size_t)turq_nq(dt) * 4u * (size_t)mpad * 16u;
}

#ifdef __HIPCC__
__device__ inline half2v as_half2(uint32_t u) { return __builtin_bit_cast(half2v, u); }
__device__ inline uint32_t as_u32(half2v h) { return __builtin_bit_cast(uint32_t, h); }

// (w & mask) | magic in ONE instruction, v_and_or_b32.  It is a VOP3 encoding, which on this ISA takes no literal
// operands; given literal constants the compiler prefers v_and_b32 + v_or_b32.  So constant masks and magics are first
// passed through an empty asm statement that pins them to a register (the wave-uniform mask to a scalar one) and that
// the optimizer cannot fold but can still hoist and share; the and/or itself stays ordinary code, for which the compiler
// then selects v_and_or_b32.  The result passes through an empty asm too, so that two of them in a row are not
// re-associated into v_and + v_and + v_or3.
//
// The instruction itself must NOT be written as inline asm.  The compiler does not know what an asm statement executes
// and keeps none of the wait states the hardware asks for around it: two between a vector instruction's write and an
// MFMA that reads the register, more between an MFMA and a vector write to its registers.  With the v_and_or_b32 in an
// asm statement, an MFMA one issue slot behind it has read the register's PREVIOUS contents (wrong sums that came and
// went with the schedule).  No asm statement in these kernels emits a vector instruction.
__device__ inline uint32_t reg_const_s(uint32_t c) {
    asm("" : "+s"(c));
    return c;
}
__device__ inline uint32_t reg_const_v(uint32_t c) {
    asm("" : "+v"(c));
    return c;
}
__device__ inline uint32_t and_or_u32(uint32_t w, uint32_t mask, uint32_t magic) {
    const uint32_t m = __builtin_constant_p(mask) ? reg_const_s(mask) : mask;
    const uint32_t g = __builtin_constant_p(magic) ? reg_const_v(magic) : magic;
    uint32_t r = (w & m) | g;
    asm("" : "+v"(r));
    return r;
}
__device__ inline half2v and_or_h2(uint32_t w, uint32_t mask, uint32_t magic) { return as_half2(and_or_u32(w, mask, magic)); }
// The instruction as inline asm, ONLY for values that feed ordinary vector arithmetic (v_pk_fma_f16, ...), never an MFMA, in a
// kernel whose MFMA results stay in their registers for the kernel's life (the prefill GEMM: its hand-placed LDS waits are
// tuned around this form, the compiler-visible one above costs it 3 %).  No MFMA reads its result and no
// register of an MFMA result is ever free for it there, so neither of the hidden wait states applies.
__device__ inline uint32_t and_or_asm(uint32_t w, uint32_t mask, uint32_t magic) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(mask), "v"(magic));
    return r;
}
__device__ inline half2v and_or_asm_h2(uint32_t w, uint32_t mask, uint32_t magic) { return as_half2(and_or_asm(w, mask, magic)); }

// fused multiply-add on a packed pair (v_pk_fma_f16): must stay fused, the intermediate product
// (base + v) * scale does not fit f16 on its own
__device__ inline half2v pk_fma(half2v a, half2v b, half2v c) { return __builtin_elementwise_fma(a, b, c); }

__device__ inline half2v splat2(_Float16 v) { return half2v{v, v}; }

__device__ inline half8v make_half8(half2v a, half2v b, half2v c, half2v d) {
    return half8v{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
}

__device__ inline float4v mfma16x16x32(half8v a, half8v b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 32-bit per-lane byte offsets of the global loads.  An offset computed (and widened to 64 bits) outside the loop reaches
// the loads as a register pair and costs a 64-bit vector add per load; one that is widened next to the load folds into the
// load's own addressing (scalar base + 32-bit lane offset).  touch() at the top of every pass makes the offsets new values
// for the compiler there, at no instruction.
struct GOff {
    uint32_t o16, o8, o4;  // 16, 8, 4 bytes per lane
    uint32_t hdr;          // 16 bytes per weight row of the tile (lane % 16)
    uint32_t aux;          // a second header offset, by format
    uint32_t frag;         // the lane's chunk inside one step of prepared activation fragments
    __device__ void touch() { asm volatile("" : "+v"(o16), "+v"(o8), "+v"(o4), "+v"(hdr), "+v"(aux), "+v"(frag)); }
};

__device__ inline uint32_t rotr32(uint32_t v, uint32_t s) { return __builtin_amdgcn_alignbit(v, v, s); }

// f32 -> bf16, round to nearest even, NaN stays a (quiet) NaN: gfx950 converts two values in one instruction
// (v_cvt_pk_bf16_f32; seven vector instructions per value when written out with integer arithmetic, which was 1 us of a
// 60 us prefill launch that stores bf16)
typedef __bf16 turq_bf16x2 __attribute__((ext_vector_type(2)));
typedef float turq_f32x2 __attribute__((ext_vector_type(2)));
__device__ inline uint32_t turq_f2bf_x2(float lo, float hi) {  // lo in bits 0..15
    const turq_bf16x2 b = __builtin_convertvector(turq_f32x2{lo, hi}, turq_bf16x2);
    uint32_t u;
    __builtin_memcpy(&u, &b, 4);
    return u;
}
__device__ inline uint16_t turq_f2bf(float f) { return (uint16_t)turq_f2bf_x2(f, 0.0f); }
// Results that are no finite numbers.  The matrix kernels compute on f16 activations: a finite f32 or bf16 input of magnitude
// 65520 or more becomes an infinity there, and what it is multiplied into comes out as an infinity or a NaN - as do inputs that
// were infinities or NaNs to begin with.  Every kernel that stores results counts the elements it stores that are not finite
// (for an f16 output: that do not fit f16) in a word of device memory, so that a host can tell that it happened
// (turq_ctx_nonfinite_count).  The word is this translation unit's own copy, one per GPU; it stops counting at 2^20.
static __device__ uint32_t turq_nonfinite_word;
// magnitudes from which a value of the output type is no finite number any more: the midpoint between the type's largest
// finite value and the next power of two rounds (to even) to an infinity
__device__ inline float turq_finite_limit(int yt) {
    return yt == TURQ_ACT_F16 ? 65520.0f : yt == TURQ_ACT_BF16 ? __uint_as_float(0x7F7F8000u) : __builtin_inff();
}
template <int YT> __device__ inline void turq_note_result(float v) {
    const float lim = turq_finite_limit(YT);
    if (__builtin_expect(!(__builtin_fabsf(v) < lim), 0)) {
        if (__hip_atomic_load(&turq_nonfinite_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (1u << 20))
            __hip_atomic_fetch_add(&turq_nonfinite_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
// the same for a run of stores: one flag per lane, one test at the end
__device__ inline void turq_note_accum(float v, float lim, uint32_t &bad) { bad |= __builtin_fabsf(v) < lim ? 0u : 1u; }
__device__ inline void turq_note_flush(uint32_t bad) {
    if (__builtin_expect(bad != 0, 0)) {
        if (__hip_atomic_load(&turq_nonfinite_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (1u << 20))
            __hip_atomic_fetch_add(&turq_nonfinite_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
// host side of it, once per translation unit whose kernels store results: adds the current device's word to *sum (and clears it)
#define TURQ_NONFINITE_READER(fn)                                                                      \
    hipError_t fn(unsigned long long *sum, int reset) {                                                \
        uint32_t v = 0;                                                                                \
        hipError_t e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(turq_nonfinite_word), sizeof v);             \
        if (e != hipSuccess) return e;                                                                 \
        *sum += v;                                                                                     \
        if (reset && v) {                                                                              \
            const uint32_t zero = 0;                                                                   \
            e = hipMemcpyToSymbol(HIP_SYMBOL(turq_nonfinite_word), &zero, sizeof zero);                \
        }                                                                                              \
        return e;                                                                                      \
    }
template <int YT> __device__ inline void turq_store_out_raw(void *y, int64_t i, float v);
template <int YT> __device__ inline void turq_store_out(void *y, int64_t i, float v) {
    turq_note_result<YT>(v);
    turq_store_out_raw<YT>(y, i, v);
}
// (without the count: for kernels that keep one flag for a run of stores)
template <int YT> __device__ inline void turq_store_out_raw(void *y, int64_t i, float v) {
    if (YT == TURQ_ACT_F32) ((float *)y)[i] = v;
    else if (YT == TURQ_ACT_BF16) ((uint16_t *)y)[i] = turq_f2bf(v);
    else {
        const _Float16 h = (_Float16)v;
        uint16_t b;
        __builtin_memcpy(&b, &h, 2);
        ((uint16_t *)y)[i] = b;
    }
}
template <int YT> __device__ inline float turq_load_out(const void *y, int64_t i) {
    if (YT == TURQ_ACT_F32) return ((const float *)y)[i];
    if (YT == TURQ_ACT_BF16) return __uint_as_float((uint32_t)((const uint16_t *)y)[i] << 16);
    const uint16_t b = ((const uint16_t *)y)[i];
    _Float16 h;
    __builtin_memcpy(&h, &b, 2);
    return (float)h;
}
// the store of a result element whose type is only known at run time; with TURQ_OUT_ACCUMULATE in yt the value is added to
// what y holds (the residual stream), in f32, and rounded once
__device__ inline void turq_store_any(void *y, int yt, int64_t i, float v) {
    const int base = yt & 0xFF;
    if (yt & TURQ_OUT_ACCUMULATE)
        v += base == TURQ_ACT_F32 ? turq_load_out<TURQ_ACT_F32>(y, i) : base == TURQ_ACT_BF16 ? turq_load_out<TURQ_ACT_BF16>(y, i) : turq_load_out<TURQ_ACT_F16>(y, i);
    if (base == TURQ_ACT_F32) turq_store_out<TURQ_ACT_F32>(y, i, v);
    else if (base == TURQ_ACT_BF16) turq_store_out<TURQ_ACT_BF16>(y, i, v);
    else turq_store_out<TURQ_ACT_F16>(y, i, v);
}
// four rows of one column, y[(row0 + i) * ldy + col] = v[i] for the rows below m: with TURQ_OUT_ACCUMULATE the four values that
// y holds are requested together and ahead of the stores (one round trip at the end of the kernel instead of four: the compiler
// cannot move a load of y across a store to y)
__device__ inline void turq_store_col4(void *y, int yt, int64_t row0, int64_t m, int64_t ldy, int64_t col, float4v v) {
    const int base = yt & 0xFF;
    float old[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (yt & TURQ_OUT_ACCUMULATE) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (row0 + i < m) {
                const int64_t at = (row0 + i) * ldy + col;
                old[i] = base == TURQ_ACT_F32 ? turq_load_out<TURQ_ACT_F32>(y, at) : base == TURQ_ACT_BF16 ? turq_load_out<TURQ_ACT_BF16>(y, at) : turq_load_out<TURQ_ACT_F16>(y, at);
            }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (row0 + i < m) turq_store_any(y, base, (row0 + i) * ldy + col, v[i] + old[i]);
}
#endif

// bytes of the prefill GEMM's fragment buffer (32-row m-tiles, 17 steps of 1 KiB per column tile)
__host__ __device__ inline size_t turq_act_prep32_bytes(int64_t m, int64_t k) {
    return (size_t)((m + 31) / 32) * (size_t)((k + 255) / 256) * 17u * 1024u;
}

// launchers (act_prep.hip, gemv_mfma.hip)
hipError_t turq_launch_act_prep32(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *frags,
                                  hipStream_t stream);
hipError_t turq_launch_rms_norm_prep32(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, const float *weight,
                                       float eps, void *frags, hipStream_t stream);
hipError_t turq_launch_silu_mul_prep32(int dtype, const float *gate, const float *up, int64_t m, int64_t n, void *frags,
                                       hipStream_t stream);
hipError_t turq_launch_act_prep(int dtype, const void *x, int x_dtype, int64_t m, int64_t k, int64_t ldx, void *frags,
                                hipStream_t stream);
hipError_t turq_launch_gemv_mfma(int dtype, const void *w_tiled, int64_t n, int64_t k, const void *xin, int x_dtype,
                                 int64_t ldx, int64_t m, bool fused, void *y, int y_dtype, int64_t ldy,
                                 const float *bias, int waves_per_group, hipStream_t stream, hipEvent_t ev_start,
                                 hipEvent_t ev_stop);
hipError_t turq_launch_gemv_multi(int dtype, int count, const void *const *w_tiled, const int64_t *n, int64_t k, const void *x,
                                  int x_dtype, int64_t ldx, int64_t m, bool fused, void *const *y, int y_dtype, const int64_t *ldy,
                                  const float *const *bias, int waves_per_group, int row_tiles_per_group, hipStream_t stream,
                                  hipEvent_t ev_start, hipEvent_t ev_stop);
// Activation rows the one-row kernel takes in one launch.  The body is written for any number M (every unpacked operand feeds
// the MFMAs of all rows).  Formats with 8 sub-blocks per tile pack two activation rows into the 16 A rows of one MFMA chain
// (turq_gemv_row1_rows() = 4); Q6_K, whose 16 sub-blocks fill the A rows, and Q8_0 take a chain per row and stop at two.
#define TURQ_ROW1_MAX_M 4
int turq_gemv_row1_rows(int dtype);
hipError_t turq_launch_gemv_gateup_frag(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *frags,
                                        int64_t m, void *y, int y_dtype, int64_t ldy, const float *bias_gate, const float *bias_up,
                                        int nwaves, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop);
// Raises a kernel's dynamic-LDS limit once per (kernel, device): the attribute belongs to the device that is current when it is
// set, and a process may hold contexts on several.
inline hipError_t turq_raise_lds_limit(const void *kernel, int bytes) {
    static std::mutex mu;
    static std::set<std::pair<const void *, int>> done;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mu);
    if (done.count({kernel, dev})) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.insert({kernel, dev});
    return e;
}

bool turq_gemv_row1_supports(int dtype);
hipError_t turq_launch_gemv_row1_gateup(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x,
                                        int x_dtype, int64_t ldx, int64_t m, void *y, int y_dtype, int64_t ldy, const float *bias_gate,
                                        const float *bias_up, int nwaves, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop,
                                        const float *norm_weight = nullptr, float norm_eps = 0.0f);
hipError_t turq_launch_gemv_row1(int dtype, int count, const void *const *w_tiled, const int64_t *n, int64_t k, const void *x,
                                 int x_dtype, int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy,
                                 const float *const *bias, int waves_per_group, int row_tiles_per_group, hipStream_t stream,
                                 hipEvent_t ev_start, hipEvent_t ev_stop, const float *norm_weight = nullptr, float norm_eps = 0.0f);
bool turq_gemv_cs_rows_ok(int row_tiles_per_group);
hipError_t turq_launch_gemv_cs(int dtype, int count, const void *const *w_tiled, const int64_t *n, int64_t k, const void *x, int x_dtype,
                               int64_t ldx, int64_t m, void *const *y, int y_dtype, const int64_t *ldy, const float *const *bias,
                               int nwaves, int row_tiles, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop);
bool turq_gemv_cs_staged_takes(int dtype_a, int dtype_b, int64_t k, int64_t m, int row_tiles);
int turq_gemv_cs_staged_second_rows(int row_tiles);
hipError_t turq_launch_gemv_cs_staged(int dtype_a, int dtype_b, int count, int second, const void *const *w_tiled, const int64_t *n,
                                      int64_t k, const void *x, int x_dtype, int64_t ldx, int64_t m, void *const *y, int y_dtype,
                                      const int64_t *ldy, const float *const *bias, int row_tiles, hipStream_t stream,
                                      hipEvent_t ev_start, hipEvent_t ev_stop);
int turq_gemv_cs_staged_gateup_tiles(int dtype, int64_t n, int64_t k, int64_t m, int64_t units);
hipError_t turq_launch_gemv_cs_staged_gateup(int dtype, const void *w_gate, const void *w_up, int64_t n, int64_t k, const void *x,
                                             int x_dtype, int64_t ldx, int64_t m, void *y, int y_dtype, int64_t ldy,
                                             const float *bias_gate, const float *bias_up, int tiles, hipStream_t stream,
                                             hipEvent_t ev_start, hipEvent_t ev_stop);
bool turq_gemv_multi_mixed_supports(int dtype_a, int dtype_b);
hipError_t turq_launch_gemv_multi_mixed(int dtype_a, int dtype_b, int count, int second, const void *const *w_tiled, const int64_t *n,
                                        int64_t k, const void *frags, int64_t m, void *const *y, int y_dtype, const int64_t *ldy,
                                        const float *const *bias, int waves_per_group, hipStream_t stream, hipEvent_t ev_start,
                                        hipEvent_t ev_stop);
bool turq_gemv_row1_mixed_supports(int dtype_a, int dtype_b);
hipError_t turq_launch_gemv_row1_mixed(int dtype_a, int dtype_b, int count, int second, const void *const *w_tiled, const int64_t *n,
                                       int64_t k, const void *x, int x_dtype, int64_t ldx, int64_t m, void *const *y, int y_dtype,
                                       const int64_t *ldy, const float *const *bias, int waves_per_group, hipStream_t stream,
                                       hipEvent_t ev_start, hipEvent_t ev_stop, const float *norm_weight = nullptr, float norm_eps = 0.0f);
// split_counters, split_partials (may be null: no launch splits its columns): TURQ_GEMM_SPLIT_COUNTER_BYTES of counters that were
// zero before the first launch that used them (every launch leaves them at zero), and turq_gemm_split_scratch(...) bytes for the
// partial tiles; launches that share either must not overlap
hipError_t turq_launch_gemm_mfma(int dtype, const void *w_tiled, int64_t n, int64_t k, const void *frags, int64_t m, void *y,
                                 int y_dtype, int64_t ldy, const float *bias, float wscale, int compute_units, hipStream_t stream,
                                 hipEvent_t ev_start, hipEvent_t ev_stop, void *split_counters = nullptr, void *split_partials = nullptr,
                                 size_t split_partial_bytes = 0);
constexpr size_t TURQ_GEMM_SPLIT_COUNTER_BYTES = 64 << 10;
// up to four weights of one format and one k in one launch of the prefill GEMM
struct TurqGemmWeights {
    const void *w[4];
    void *y[4];
    const float *bias[4];
    int64_t n[4], ldy[4];
    float wscale[4];
    int count;
};
hipError_t turq_launch_gemm_mfma_group(int dtype, const TurqGemmWeights &ws, int64_t k, const void *frags, int64_t m, int y_dtype,
                                       int compute_units, hipStream_t stream, hipEvent_t ev_start, hipEvent_t ev_stop,
                                       void *split_counters = nullptr, void *split_partials = nullptr, size_t split_partial_bytes = 0);
// the workgroup tile the launch rules pick (0: no kernel for the format)
int turq_gemm_form(int dtype, int64_t n, int64_t k, int64_t m, int compute_units);
// the launch the tile rules would make for these rows: its workgroups and the share of its CU rounds it keeps busy (x the wide
// tile's gain)
double turq_gemm_fill(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int64_t *wgs_out);
bool turq_gemm_low_two_groups(int64_t n, int64_t k, int64_t m, int split, int compute_units);
// bytes of partial tiles a launch of this shape wants for splitting its columns, 0 if it does not split; form_out / split_out
// (may be null): the tile (3: wide, 4: low) and the number of parts
size_t turq_gemm_split_scratch(int dtype, int64_t n, int64_t k, int64_t m, int compute_units, int *form_out, int *split_out);
