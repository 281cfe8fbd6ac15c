// The tiled HBM layout of quantized weights (TURQ_LAYOUT_TILED) and its mapping to GGUF bytes.
//
// Why a second layout: the MFMA kernels give weight row r of a 16-row tile to lanes r, r+16, r+32,
// r+48 of a wave (lane = r + 16*g).  In GGUF order those lanes would touch 16 different rows per
// load instruction; in the tiled order every load instruction of a wave reads one contiguous,
// lane-linear plane (lane L reads bytes [16*L, 16*L+16) of a 1 KiB plane).  The total size is
// unchanged (no padding inside a block; rows are padded to a multiple of 16 and, for Q8_0, columns
// to a multiple of 256 with zero blocks).
//
// Geometry shared by all formats
//   row tile rt = row / 16, r = row % 16;  column tile b = column / 256;  lane L = r + 16*g, g = 0..3
//   tile (rt, b) starts at byte (rt * ntile_cols + b) * kTileBytes
//   K-quants: lane (r, g) owns elements 64*g .. 64*g+63 of super-block b of row r, and MFMA step
//             q = 0..7 consumes its elements 64*g + 8*q + j, j = 0..7 (operand slot j)
//   Q8_0:     MFMA step q consumes block q of the 8 blocks in the tile; lane (r, g) owns its
//             elements 8*g + j
//
// Q4_K tile, 2304 B:   [QA 1024][QB 1024][HDR 256]
//   lane dword i (i = 0..3 in QA at 16*L + 4*i, i = 4..7 in QB) holds the 8 nibbles of MFMA step i:
//   slot j sits at bit 4 * kNibblePos[j], kNibblePos = {0, 4, 1, 5, 2, 6, 3, 7}, so that
//   (w & 0x000F000F) is slots (0,1), (w & 0x00F000F0) slots (2,3), and the same masks on w >> 8
//   give slots (4,5) and (6,7), each pair already in the two halves of a packed-f16 register.
//   HDR row r (16 B): u16 d, u16 dmin, then four 24-bit groups, group g at bit 24*g:
//   sc[2g] | m[2g] << 6 | sc[2g+1] << 12 | m[2g+1] << 18  (the 6-bit scales / mins of the two
//   sub-blocks lane (r, g) owns).
// Q5_K tile, 2816 B:   [QA 1024][QB 1024][QH 512][HDR 256]
//   QA/QB/HDR as Q4_K.  QH: lane L has two dwords at 8*L.  With v = 4*i + t the packed register
//   t = 0..3 of step i (slots 2t, 2t+1), u = v >> 1: for even t the high bits of its two elements
//   sit in H0 at bits (4 + u) % 32 and (20 + u) % 32, for odd t in H1 at bits (8 + u) % 32 and
//   (24 + u) % 32, so a rotate right by u drops them on top of the nibbles selected above.
// Q6_K tile, 3360 B:   [QLA 1024][QLB 1024][QH 1024][SC 256][D 32]
//   low nibbles: lane dword i holds MFMA step i, slot j at bit kQ6NibbleBit[j] (4 bits, wrapping
//   past bit 31), kQ6NibbleBit = {2, 18, 6, 22, 10, 26, 14, 30}: masks 0x003C003C / 0x03C003C0 on w
//   and on rotr(w, 8) give the four packed registers with the nibble in mantissa bits 2..5 or 6..9.
//   high 2-bit fields: lane dwords H0..H3 at QH + 16*L; dword i >> 1 holds the 16 fields of steps
//   2*(i>>1) and 2*(i>>1)+1.  With f = (i & 1) * 8 + j, rp = f >> 1, s = f & 1 the field sits at bit
//   (6 + 2 * (rp & 1) + 16 * s + 4 * (rp >> 1)) % 32: a rotate right by 0, 4, 8 or 12 drops two
//   registers' worth of fields on mantissa bits 6..7 (rp even) or 8..9 (rp odd) of both halves.
//   SC: lane L has 4 int8 at 4*L: scales[4g .. 4g+3] of row r.   D: row r has u16 d at 2*r.
// Q8_0 tile, 4352 B:   [P0 1024][P1 1024][P2 1024][P3 1024][D 256]
//   plane i, lane L, 16 B = dwords (2i, lo), (2i, hi), (2i+1, lo), (2i+1, hi): block q's elements
//   8g + j as bytes (q + 128) at byte kByteOrder[j % 4] of dword (j / 4), kByteOrder = {0, 2, 1, 3}.
//   D: row r has 8 u16 at 16*r (block q's scale at index q).
#pragma once

#include "common.h"

template <int DT> struct TiledFmt;

template <> struct TiledFmt<TURQ_Q4_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 144, kTileCols = 256, kTileBytes = 2304;
    static constexpr int kQA = 0, kQB = 1024, kHDR = 2048;
};
template <> struct TiledFmt<TURQ_Q5_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 176, kTileCols = 256, kTileBytes = 2816;
    static constexpr int kQA = 0, kQB = 1024, kQH = 2048, kHDR = 2560;
};
template <> struct TiledFmt<TURQ_Q6_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 210, kTileCols = 256, kTileBytes = 3360;
    static constexpr int kQLA = 0, kQLB = 1024, kQH = 2048, kSC = 3072, kD = 3328;
};
template <> struct TiledFmt<TURQ_Q8_0> {
    static constexpr int kBlockElems = 32, kBlockBytes = 34, kTileCols = 256, kTileBytes = 4352;
    static constexpr int kD = 4096;
};

__host__ __device__ inline int64_t turq_tile_rows(int64_t n) { return (n + 15) / 16; }
__host__ __device__ inline int64_t turq_tile_cols(int64_t k) { return (k + 255) / 256; }

__host__ __device__ inline int turq_tile_bytes(int dt) {
    switch (dt) {
    case TURQ_Q4_K: return 2304;
    case TURQ_Q5_K: return 2816;
    case TURQ_Q6_K: return 3360;
    case TURQ_Q8_0: return 4352;
    default: return 0;
    }
}

// ---- bit helpers on a little-endian byte buffer viewed as 32-bit words ----
__host__ __device__ inline uint32_t turq_ld32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
__host__ __device__ inline void turq_st32(uint8_t *p, uint32_t v) {
    p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24);
}
__host__ __device__ inline uint32_t turq_rotl32(uint32_t v, int s) { s &= 31; return s ? (v << s) | (v >> (32 - s)) : v; }
__host__ __device__ inline uint32_t turq_rotr32(uint32_t v, int s) { s &= 31; return s ? (v >> s) | (v << (32 - s)) : v; }
// `bits`-wide field at bit `pos` (wrapping past bit 31)
__host__ __device__ inline uint32_t turq_get_field(uint32_t w, int pos, int bits) {
    return turq_rotr32(w, pos) & ((1u << bits) - 1u);
}
__host__ __device__ inline uint32_t turq_set_field(uint32_t w, int pos, int bits, uint32_t v) {
    const uint32_t mask = turq_rotl32((1u << bits) - 1u, pos);
    return (w & ~mask) | (turq_rotl32(v, pos) & mask);
}

// slot j of a Q4_K / Q5_K step dword sits at bit 4 * kNibblePos[j]
__host__ __device__ inline int turq_q4_nibble_bit(int j) {
    // j: 0 1 2 3 4 5 6 7  ->  nibble index 0 4 1 5 2 6 3 7
    return 4 * (((j & 1) << 2) | (j >> 1));
}
// slot j of a Q6_K low-nibble step dword
__host__ __device__ inline int turq_q6_nibble_bit(int j) {
    // j: 0 1 2 3 4 5 6 7 -> 2 18 6 22 10 26 14 30
    return 2 + 16 * (j & 1) + 4 * (j >> 1);
}
// Q6_K high fields: lane dword hd = i >> 1 (i = MFMA step) holds 16 two-bit fields.  Field index
// f = (i & 1) * 8 + j.  Register pair index rp = f >> 1 (0..7), s = f & 1 selects the half.
// A rotate right by 4 * (rp >> 1) leaves the pair on bits 6..7 (rp even) or 8..9 (rp odd) of the
// half s, i.e. it is stored at bit (6 + 2 * (rp & 1) + 16 * s + 4 * (rp >> 1)) % 32.
__host__ __device__ inline int turq_q6_high_bit(int i, int j) {
    const int f = (i & 1) * 8 + j;
    const int rp = f >> 1, s = f & 1;
    return (6 + 2 * (rp & 1) + 16 * s + 4 * (rp >> 1)) & 31;
}
// Q5_K high bits: register v = 4*i + t, u = v >> 1, slot half s: H[t & 1] bit (4 + 4*(t&1) + u + 16*s) % 32
__host__ __device__ inline int turq_q5_high_bit(int i, int j) {
    const int t = j >> 1, s = j & 1;
    const int u = (4 * i + t) >> 1;
    return (4 + 4 * (t & 1) + u + 16 * s) & 31;
}

// 6-bit scales / mins of a native Q4_K / Q5_K block
__host__ __device__ inline void turq_unpack_k4(const uint8_t *q, uint32_t sc[8], uint32_t mn[8]) {
    for (int j = 0; j < 4; j++) {
        sc[j] = q[j] & 63u;
        mn[j] = q[j + 4] & 63u;
        sc[j + 4] = (q[j + 8] & 0x0Fu) | ((uint32_t)(q[j] >> 6) << 4);
        mn[j + 4] = (uint32_t)(q[j + 8] >> 4) | ((uint32_t)(q[j + 4] >> 6) << 4);
    }
}
__host__ __device__ inline void turq_pack_k4(const uint32_t sc[8], const uint32_t mn[8], uint8_t *q) {
    for (int j = 0; j < 4; j++) {
        q[j] = (uint8_t)(sc[j] | ((sc[j + 4] >> 4) << 6));
        q[j + 4] = (uint8_t)(mn[j] | ((mn[j + 4] >> 4) << 6));
        q[j + 8] = (uint8_t)((sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4));
    }
}

// Element e (0..63) of lane group g in a K-quant super-block is native element 64*g + e.
// Native Q4_K / Q5_K: element E lives in qs[32 * (E / 64) + E % 32], low nibble if (E / 32) even.
__host__ __device__ inline uint32_t turq_native_nibble_q45(const uint8_t *qs, int E) {
    const uint8_t b = qs[32 * (E >> 6) + (E & 31)];
    return ((E >> 5) & 1) ? (b >> 4) : (b & 0xF);
}
__host__ __device__ inline void turq_native_set_nibble_q45(uint8_t *qs, int E, uint32_t v) {
    uint8_t &b = qs[32 * (E >> 6) + (E & 31)];
    b = ((E >> 5) & 1) ? (uint8_t)((b & 0x0F) | (v << 4)) : (uint8_t)((b & 0xF0) | v);
}
// Native Q6_K: E -> (half, quarter, l): ql[64*half + 32*(quarter&1) + l] nibble (quarter>>1), qh[32*half + l] >> 2*quarter
__host__ __device__ inline void turq_native_q6_pos(int E, int &ql_idx, int &ql_hi, int &qh_idx, int &qh_shift) {
    const int half = E >> 7, r = E & 127, quarter = r >> 5, l = r & 31;
    ql_idx = 64 * half + 32 * (quarter & 1) + l;
    ql_hi = quarter >> 1;
    qh_idx = 32 * half + l;
    qh_shift = 2 * quarter;
}

// ---- one native block <-> its place in the tiled buffer ----
// `tile` points at the start of tile (rt, b); r is the row inside the tile.

template <int DT> struct TileBlock;

template <> struct TileBlock<TURQ_Q4_K> {
    using F = TiledFmt<TURQ_Q4_K>;
    __host__ __device__ static void pack_hdr(const uint8_t *nat, uint8_t *hdr) {
        hdr[0] = nat[0]; hdr[1] = nat[1]; hdr[2] = nat[2]; hdr[3] = nat[3];
        uint32_t sc[8], mn[8];
        turq_unpack_k4(nat + 4, sc, mn);
        uint32_t wds[3] = {0, 0, 0};
        for (int g = 0; g < 4; g++) {
            const uint32_t G = sc[2 * g] | (mn[2 * g] << 6) | (sc[2 * g + 1] << 12) | (mn[2 * g + 1] << 18);
            const int bit = 24 * g;
            wds[bit >> 5] |= G << (bit & 31);
            if ((bit & 31) > 8) wds[(bit >> 5) + 1] |= G >> (32 - (bit & 31));
        }
        for (int i = 0; i < 3; i++) turq_st32(hdr + 4 + 4 * i, wds[i]);
    }
    __host__ __device__ static void unpack_hdr(const uint8_t *hdr, uint8_t *nat) {
        nat[0] = hdr[0]; nat[1] = hdr[1]; nat[2] = hdr[2]; nat[3] = hdr[3];
        uint32_t wds[4] = {turq_ld32(hdr + 4), turq_ld32(hdr + 8), turq_ld32(hdr + 12), 0};
        uint32_t sc[8], mn[8];
        for (int g = 0; g < 4; g++) {
            const int bit = 24 * g;
            uint32_t G = wds[bit >> 5] >> (bit & 31);
            if ((bit & 31) > 8) G |= wds[(bit >> 5) + 1] << (32 - (bit & 31));
            G &= 0xFFFFFFu;
            sc[2 * g] = G & 63; mn[2 * g] = (G >> 6) & 63; sc[2 * g + 1] = (G >> 12) & 63; mn[2 * g + 1] = (G >> 18) & 63;
        }
        turq_pack_k4(sc, mn, nat + 4);
    }
    __host__ __device__ static void tile(const uint8_t *nat, uint8_t *tile, int r) {
        pack_hdr(nat, tile + F::kHDR + 16 * r);
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            for (int i = 0; i < 8; i++) {
                uint32_t w = 0;
                for (int j = 0; j < 8; j++)
                    w |= turq_native_nibble_q45(nat + 16, 64 * g + 8 * i + j) << turq_q4_nibble_bit(j);
                turq_st32(tile + (i < 4 ? F::kQA : F::kQB) + 16 * L + 4 * (i & 3), w);
            }
        }
    }
    __host__ __device__ static void untile(const uint8_t *tile, int r, uint8_t *nat) {
        unpack_hdr(tile + F::kHDR + 16 * r, nat);
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            for (int i = 0; i < 8; i++) {
                const uint32_t w = turq_ld32(tile + (i < 4 ? F::kQA : F::kQB) + 16 * L + 4 * (i & 3));
                for (int j = 0; j < 8; j++)
                    turq_native_set_nibble_q45(nat + 16, 64 * g + 8 * i + j, (w >> turq_q4_nibble_bit(j)) & 0xF);
            }
        }
    }
};

template <> struct TileBlock<TURQ_Q5_K> {
    using F = TiledFmt<TURQ_Q5_K>;
    __host__ __device__ static void tile(const uint8_t *nat, uint8_t *tile, int r) {
        TileBlock<TURQ_Q4_K>::pack_hdr(nat, tile + F::kHDR + 16 * r);
        const uint8_t *qh = nat + 16, *qs = nat + 48;
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            uint32_t H[2] = {0, 0};
            for (int i = 0; i < 8; i++) {
                uint32_t w = 0;
                for (int j = 0; j < 8; j++) {
                    const int E = 64 * g + 8 * i + j;
                    w |= turq_native_nibble_q45(qs, E) << turq_q4_nibble_bit(j);
                    const uint32_t hb = (qh[E & 31] >> (E >> 5)) & 1u;
                    H[(j >> 1) & 1] |= hb << turq_q5_high_bit(i, j);
                }
                turq_st32(tile + (i < 4 ? F::kQA : F::kQB) + 16 * L + 4 * (i & 3), w);
            }
            turq_st32(tile + F::kQH + 8 * L, H[0]);
            turq_st32(tile + F::kQH + 8 * L + 4, H[1]);
        }
    }
    __host__ __device__ static void untile(const uint8_t *tile, int r, uint8_t *nat) {
        TileBlock<TURQ_Q4_K>::unpack_hdr(tile + F::kHDR + 16 * r, nat);
        uint8_t *qh = nat + 16, *qs = nat + 48;
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            const uint32_t H[2] = {turq_ld32(tile + F::kQH + 8 * L), turq_ld32(tile + F::kQH + 8 * L + 4)};
            for (int i = 0; i < 8; i++) {
                const uint32_t w = turq_ld32(tile + (i < 4 ? F::kQA : F::kQB) + 16 * L + 4 * (i & 3));
                for (int j = 0; j < 8; j++) {
                    const int E = 64 * g + 8 * i + j;
                    turq_native_set_nibble_q45(qs, E, (w >> turq_q4_nibble_bit(j)) & 0xF);
                    const uint32_t hb = (H[(j >> 1) & 1] >> turq_q5_high_bit(i, j)) & 1u;
                    uint8_t &b = qh[E & 31];
                    b = (uint8_t)((b & ~(1u << (E >> 5))) | (hb << (E >> 5)));
                }
            }
        }
    }
};

template <> struct TileBlock<TURQ_Q6_K> {
    using F = TiledFmt<TURQ_Q6_K>;
    __host__ __device__ static void tile(const uint8_t *nat, uint8_t *tile, int r) {
        const uint8_t *ql = nat, *qh = nat + 128, *sc = nat + 192;
        tile[F::kD + 2 * r] = nat[208];
        tile[F::kD + 2 * r + 1] = nat[209];
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            for (int c = 0; c < 4; c++) tile[F::kSC + 4 * L + c] = sc[4 * g + c];
            uint32_t H[4] = {0, 0, 0, 0};
            for (int i = 0; i < 8; i++) {
                uint32_t w = 0;
                for (int j = 0; j < 8; j++) {
                    int li, lhi, hi, hs;
                    turq_native_q6_pos(64 * g + 8 * i + j, li, lhi, hi, hs);
                    const uint32_t nib = lhi ? (ql[li] >> 4) : (ql[li] & 0xF);
                    const uint32_t h2 = (qh[hi] >> hs) & 3u;
                    w = turq_set_field(w, turq_q6_nibble_bit(j), 4, nib);
                    H[i >> 1] = turq_set_field(H[i >> 1], turq_q6_high_bit(i, j), 2, h2);
                }
                turq_st32(tile + (i < 4 ? F::kQLA : F::kQLB) + 16 * L + 4 * (i & 3), w);
            }
            for (int c = 0; c < 4; c++) turq_st32(tile + F::kQH + 16 * L + 4 * c, H[c]);
        }
    }
    __host__ __device__ static void untile(const uint8_t *tile, int r, uint8_t *nat) {
        uint8_t *ql = nat, *qh = nat + 128, *sc = nat + 192;
        nat[208] = tile[F::kD + 2 * r];
        nat[209] = tile[F::kD + 2 * r + 1];
        for (int g = 0; g < 4; g++) {
            const int L = r + 16 * g;
            for (int c = 0; c < 4; c++) sc[4 * g + c] = tile[F::kSC + 4 * L + c];
            uint32_t H[4];
            for (int c = 0; c < 4; c++) H[c] = turq_ld32(tile + F::kQH + 16 * L + 4 * c);
            for (int i = 0; i < 8; i++) {
                const uint32_t w = turq_ld32(tile + (i < 4 ? F::kQLA : F::kQLB) + 16 * L + 4 * (i & 3));
                for (int j = 0; j < 8; j++) {
                    int li, lhi, hi, hs;
                    turq_native_q6_pos(64 * g + 8 * i + j, li, lhi, hi, hs);
                    const uint32_t nib = turq_get_field(w, turq_q6_nibble_bit(j), 4);
                    const uint32_t h2 = turq_get_field(H[i >> 1], turq_q6_high_bit(i, j), 2);
                    ql[li] = lhi ? (uint8_t)((ql[li] & 0x0F) | (nib << 4)) : (uint8_t)((ql[li] & 0xF0) | nib);
                    qh[hi] = (uint8_t)((qh[hi] & ~(3u << hs)) | (h2 << hs));
                }
            }
        }
    }
};

// Q8_0: `tile` points at tile (rt, tb) which holds blocks 8*tb .. 8*tb+7 of 16 rows; q = block % 8.
template <> struct TileBlock<TURQ_Q8_0> {
    using F = TiledFmt<TURQ_Q8_0>;
    __host__ __device__ static int byte_of(int q, int g, int j, int r) {
        const int L = r + 16 * g;
        const int dw = (q & 1) * 2 + (j >> 2);           // dword inside the lane's 16 bytes
        const int c = ((j & 1) << 1) | ((j >> 1) & 1);   // byte order {0, 2, 1, 3}
        return 1024 * (q >> 1) + 16 * L + 4 * dw + c;
    }
    __host__ __device__ static void tile(const uint8_t *nat, uint8_t *tile, int r, int q) {
        tile[F::kD + 16 * r + 2 * q] = nat[0];
        tile[F::kD + 16 * r + 2 * q + 1] = nat[1];
        for (int g = 0; g < 4; g++)
            for (int j = 0; j < 8; j++) tile[byte_of(q, g, j, r)] = (uint8_t)(nat[2 + 8 * g + j] ^ 0x80);
    }
    __host__ __device__ static void untile(const uint8_t *tile, int r, int q, uint8_t *nat) {
        nat[0] = tile[F::kD + 16 * r + 2 * q];
        nat[1] = tile[F::kD + 16 * r + 2 * q + 1];
        for (int g = 0; g < 4; g++)
            for (int j = 0; j < 8; j++) nat[2 + 8 * g + j] = (uint8_t)(tile[byte_of(q, g, j, r)] ^ 0x80);
    }
};

// Rebuild native block `b` (index along the row, in units of the format's block) of row `row`.
template <int DT>
__host__ __device__ inline void turq_untile_block(const uint8_t *w, int64_t k, int64_t row, int64_t b, uint8_t *nat) {
    const int64_t ntc = turq_tile_cols(k);
    const int64_t rt = row >> 4;
    const int r = (int)(row & 15);
    if constexpr (DT == TURQ_Q8_0) {
        const uint8_t *tile = w + (rt * ntc + (b >> 3)) * TiledFmt<DT>::kTileBytes;
        TileBlock<DT>::untile(tile, r, (int)(b & 7), nat);
    } else {
        const uint8_t *tile = w + (rt * ntc + b) * TiledFmt<DT>::kTileBytes;
        TileBlock<DT>::untile(tile, r, nat);
    }
}

// Place native block `b` of row `row` into the tiled buffer (which must start zero-filled).
template <int DT>
__host__ __device__ inline void turq_tile_block(const uint8_t *nat, uint8_t *w, int64_t k, int64_t row, int64_t b) {
    const int64_t ntc = turq_tile_cols(k);
    const int64_t rt = row >> 4;
    const int r = (int)(row & 15);
    if constexpr (DT == TURQ_Q8_0) {
        uint8_t *tile = w + (rt * ntc + (b >> 3)) * TiledFmt<DT>::kTileBytes;
        TileBlock<DT>::tile(nat, tile, r, (int)(b & 7));
    } else {
        uint8_t *tile = w + (rt * ntc + b) * TiledFmt<DT>::kTileBytes;
        TileBlock<DT>::tile(nat, tile, r);
    }
}
