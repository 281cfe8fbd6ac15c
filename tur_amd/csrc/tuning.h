// Every environment switch that changes which kernel a call takes, or how it is launched, in ONE table.
//
// The rules in mfma_dispatch.cpp and at the end of gemm_mfma.hip choose kernels, tiles, splits and wave counts from the shape of
// a call and the size of the device; their thresholds were measured on MI355X.  Each of the switches below overrides one rule,
// for A/B timing and for tests that must reach a kernel the rule would not pick.  None is needed in production.  The
// environment is read ONCE per process, when the first context is created (turq_tuning() below); a process that runs with any
// of them set says so in one line on stderr at that moment, and turq_tuning_describe() lists the values a process runs with.
#pragma once
#include <cstddef>

// X(field, "ENVIRONMENT NAME", kind, default, "what it overrides")
//   kind INT : the variable's integer value, or the default when it is unset
//   kind FLAG: true when the variable is set at all
//   kind OFF : true when the variable is set to 0 (the feature is switched off)
//   kind TRI : -1 when unset, else 0 / 1
#define TURQ_TUNING_TABLE(X)                                                                                                              \
    X(gemv_waves, "TURQ_GEMV_WAVES", INT, 0, "waves per workgroup of the decode kernels (1 .. 16) instead of the rule's choice")            \
    X(gemv_no_row1, "TURQ_GEMV_NO_ROW1", FLAG, 0, "never take the one-row kernels (gemv_row1.hip); the general skinny kernel runs instead") \
    X(row1_m, "TURQ_ROW1_M", INT, 4, "most activation rows the one-row kernels take (1 .. 4)")                                              \
    X(row1_tpw, "TURQ_ROW1_TPW", INT, 0, "column tiles per wave of the one-row kernels")                                                    \
    X(row1_r, "TURQ_ROW1_R", INT, 0, "row tiles per workgroup of the one-row kernels (1 or 2)")                                             \
    X(row1_p, "TURQ_ROW1_P", INT, 0, "column tiles in flight per wave of the one-row kernels (2 or 3)")                                     \
    X(cs, "TURQ_CS", INT, -1, "0: never take the column-split kernel on prepared fragments (gemv_cs.hip)")                                  \
    X(cs_rg, "TURQ_CS_RG", INT, 0, "row tiles per workgroup of the column-split and staged kernels")                                        \
    X(cs_staged, "TURQ_CS_STAGED", INT, -1, "0: never take the kernels that stage the rows themselves (gemv_cs_staged.h)")                  \
    X(cs_staged_min_m, "TURQ_CS_STAGED_MIN_M", INT, 3, "fewest rows the staged kernels take")                                               \
    X(cs_staged_max_m, "TURQ_CS_STAGED_MAX_M", INT, 32, "most rows the staged kernels take")                                                \
    X(cs_waves, "TURQ_CS_WAVES", INT, 0, "waves per workgroup of the column-split kernel (1 .. 8)")                                         \
    X(gemv_rowtiles, "TURQ_GEMV_ROWTILES", INT, 0, "row tiles per set of fragments of the general skinny kernel (1 or 2)")                  \
    X(gemv_no_fuse, "TURQ_GEMV_NO_FUSE", FLAG, 0, "always prepare the activation fragments in a launch of their own")                       \
    X(gemv_no_mixed, "TURQ_GEMV_NO_MIXED", FLAG, 0, "never join a second format into one decode launch (q, k Q4_K + v Q6_K)")               \
    X(gateup_no_frag, "TURQ_GATEUP_NO_FRAG", FLAG, 0, "turq_qmatmul_gate_up at 17 .. 32 rows: leave the prepared-fragment route out")       \
    X(rows_in_chunks_off, "TURQ_ROWS_IN_CHUNKS", OFF, 0, "33 .. 64 rows never go through the decode kernels in two chunks")                 \
    X(norm_fused_off, "TURQ_NORM_FUSED", OFF, 0, "turq_norm_*: always normalise into scratch first")                                        \
    X(mlp_prefill_off, "TURQ_MLP_PREFILL", OFF, 0, "turq_mlp above 32 rows: separate calls instead of the fused middle kernel")             \
    X(gemm_no_side, "TURQ_GEMM_NO_SIDE", FLAG, 0, "turq_qmatmul_multi above 32 rows: every launch on the context's stream")                 \
    X(gemm_merge, "TURQ_GEMM_MERGE", INT, -1, "gate / up as one prefill launch: 0 never, 2 always (default: the rule)")                     \
    X(gemm_grid_2x2, "TURQ_GEMM_GRID_2X2", FLAG, 0, "Q5_K / Q6_K prefill tiles on the 2 x 2 wave grid")                                     \
    X(gemm_wide, "TURQ_GEMM_WIDE", TRI, -1, "prefill: the wide tile 128 x 256 always (1) or never (0)")                                     \
    X(gemm_low, "TURQ_GEMM_LOW", TRI, -1, "prefill: the low tile 64 x 128 always (1) or never (0)")                                         \
    X(gemm_split, "TURQ_GEMM_SPLIT", INT, -1, "prefill: workgroups per tile that share its columns (0 / 1: never split)")                   \
    X(gemm_split_form, "TURQ_GEMM_SPLIT_FORM", INT, 0, "prefill: tile of a forced split (3 wide, 4 low)")                                   \
    X(gemm_kgroups, "TURQ_GEMM_KGROUPS", INT, 0, "prefill low tile: 1 four waves, 2 eight waves as two groups")                             \
    X(prefetch_wgs, "TURQ_PREFETCH_WGS", INT, 0, "workgroups of turq_weight_prefetch (1 .. 4096)")                                          \
    X(prefetch_depth, "TURQ_PREFETCH_DEPTH", INT, 0, "4 KiB chunks in flight per wave of turq_weight_prefetch (1 .. 4)")

struct TurqTuning {
#define TURQ_TUNING_FIELD_INT(f, d) int f = d;
#define TURQ_TUNING_FIELD_TRI(f, d) int f = d;
#define TURQ_TUNING_FIELD_FLAG(f, d) bool f = false;
#define TURQ_TUNING_FIELD_OFF(f, d) bool f = false;
#define X(f, env, kind, d, doc) TURQ_TUNING_FIELD_##kind(f, d)
    TURQ_TUNING_TABLE(X)
#undef X
#undef TURQ_TUNING_FIELD_INT
#undef TURQ_TUNING_FIELD_TRI
#undef TURQ_TUNING_FIELD_FLAG
#undef TURQ_TUNING_FIELD_OFF
    int overrides = 0;  // how many of the variables were set when the environment was read
};

// the switches of this process (the environment is read at the first call; turq_ctx_create makes it)
const TurqTuning &turq_tuning();
