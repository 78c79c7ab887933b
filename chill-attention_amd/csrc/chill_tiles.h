// Static MI355X tile table: (mask id, head dim, dtype, pass) -> tile shape.  It replaces the
// reference's per-GPU default tables and Triton autotune spaces (chill_attention/autotune.py:11-119,
// 129-240).  The functions are constexpr so the kernel launchers instantiate exactly the shapes the
// table reports through chill_tile_config().
//
// rows     = resident rows per workgroup (32 per wave): query rows in the forward and dQ passes,
//            key rows in the dK/dV pass;
// streamed = rows of one streamed LDS tile: keys in forward / dQ, queries in dK/dV.
#pragma once

#include "chill_params.h"

// Build-time overrides for the tile sweep (chill_attention/tune.py builds one library per candidate
// shape): 16-bit inputs with head dim <= 128 only.  Without them the table below is what ships.
#ifndef CHILL_TUNE_FWD_WAVES
#define CHILL_TUNE_FWD_WAVES 0
#endif
#ifndef CHILL_TUNE_FWD_STREAMED
#define CHILL_TUNE_FWD_STREAMED 0
#endif
#ifndef CHILL_TUNE_FWD_SMALL
#define CHILL_TUNE_FWD_SMALL 1
#endif
#ifndef CHILL_TUNE_FWD_STAGES
#define CHILL_TUNE_FWD_STAGES 0
#endif
#ifndef CHILL_TUNE_DQ_STAGES
#define CHILL_TUNE_DQ_STAGES 0
#endif
#ifndef CHILL_TUNE_DQ_WAVES
#define CHILL_TUNE_DQ_WAVES 0
#endif
#ifndef CHILL_TUNE_DQ_STREAMED
#define CHILL_TUNE_DQ_STREAMED 0
#endif
#ifndef CHILL_TUNE_DKDV_WAVES
#define CHILL_TUNE_DKDV_WAVES 0
#endif

// 1: the 8-wave forward of 16-bit inputs at head dim 128 streams 64-key tiles through four stages,
// the shape fwd_q_tile_fast and its generated loop are written for; 0: the shape before it (128-key
// tiles, two stages, fwd_q_tile).
#ifndef CHILL_FWD_FAST
#define CHILL_FWD_FAST 1
#endif

namespace chill {

constexpr int elem_bytes(int dtype) { return dtype == CHILL_F32 ? 4 : 2; }

// Forward LDS stage: a K tile padded for row-wise reads and a V tile padded for transposed reads
// (pads as in PaddedTile, chill_device.h).
constexpr int fwd_stage_bytes(int streamed, int D, int dtype) {
    const int rb = D * elem_bytes(dtype);
    const int vpad = dtype == CHILL_F32 ? 32 : (rb >= 128 ? 64 : 0);
    return streamed * (rb + 16) + streamed * (rb + vpad);
}

// Masks whose rows see a narrow band of keys: a q-tile is a short loop, and the time a workgroup
// spends before and after it (loading Q and the first K/V tile, storing O) is a large part of its
// life.  They get workgroups of four waves with a two-stage ring, two of which share a CU, so that one
// computes while the other loads or stores (measured: sliding window forward -22 %, dQ -16 %;
// chunkwise forward -5 %, dQ -14 %; on the causal workload the same shape re-reads K and V twice as
// often and is 1-2 % slower).
constexpr bool mask_is_banded(int mask_id) {
    return mask_id == CHILL_MASK_SLIDING_WINDOW || mask_id == CHILL_MASK_CHUNKWISE;
}
// The most keys a row of such a mask sees (`a0`, `a1` = the mask's first two arguments: left and right context, or
// chunk size and chunks looked back at); kWholeSequence for the other masks.  A wide band is a long loop again:
// the forward and dK/dV then take the shapes of the masks that are not banded, from the widths named at
// fwd_takes_short_row and dkdv_regs_serves_band on.
constexpr long long kWholeSequence = 1ll << 40;
constexpr long long mask_band_keys(int mask_id, long long a0, long long a1) {
    return mask_id == CHILL_MASK_SLIDING_WINDOW ? a0 + a1 + 1 : mask_id == CHILL_MASK_CHUNKWISE ? a0 * (a1 + 1) : kWholeSequence;
}
// (a banded mask of which only the id is known is taken to be narrow)
constexpr long long kNarrowBand = 1;

// Sequence lengths up to which the 4-wave shape also wins at head dim 128 for masks that are not banded
// (measured on causal and full masks, B8 H4 .. H16: forward -16 % at T = 512 and 1024, +20 % at 2085;
// dQ -24 % at 512, -14 % at 2048 and 4042, -5 % at 4096, +-1 % at 8192, where its extra K / V reads cost
// the neighbouring kernels more than it gains).  T = kLongSequence selects the long-sequence row.
constexpr int kLongSequence = 0x7fffffff;
constexpr int kFwdShortSequence = 1024;
constexpr int kFwdShortSequenceFull = 768;
constexpr int kDqShortSequence = 4096;
// The same shape is taken when the 8-wave one would leave CUs without a workgroup (B1 H8 T8192 causal:
// forward -7 %, dQ -17 %; with twice as many heads the 8-wave shape wins again).
constexpr int kComputeUnits = 256;
// (forward: only dQ still takes it; the 8-wave forward with its generated loop is 23 % faster than the 4-wave
// one at B1 H8 T8192)
// Banded masks take it while a row sees fewer than kFwdWideBand keys (measured at head dim 128, T = 8192 and 16384,
// the 8-wave shape against this one: sliding windows of 512 / 1024 / 2048 / 4096 keys +9 / -12 / -18 / -18 %,
// chunkwise 1024 x 2 -17 %, 128 x 3 +2 %).
constexpr int kFwdWideBand = 1024;
constexpr bool fwd_takes_short_row(int mask_id, long long band_keys, long long batch_heads, int T) {
    (void)batch_heads;
    // (under a full mask the 8-wave shape, whose loop is predicate-free from its first tile on, wins from 769 keys on:
    // B16 H16 T = 1024 / 1000 -12 / -7 %, T = 768 / 512 +2 / -1 %; causal T = 1024 / 768 / 512 +3 / +41 / +23 %)
    return T <= (mask_id == CHILL_MASK_FULL ? kFwdShortSequenceFull : kFwdShortSequence) ||
           (mask_is_banded(mask_id) && band_keys < kFwdWideBand);
}
constexpr bool dq_takes_short_row(long long batch_heads, int T) {
    return T <= kDqShortSequence || batch_heads * ((T + 255) / 256) <= kComputeUnits;
}

// Forward.  16-bit inputs at head dim 128: 8 waves (256 query rows), streamed tiles of 128 keys (half
// the barriers per key); narrow bands (fwd_takes_short_row), head dims <= 64 and short sequences: 4 waves, 64 keys, 2
// stages, two or three workgroups per CU (prefix-LM at D = 64: forward -14 %; causal at D = 16 .. 64:
// -5 .. -8 %).
constexpr int fwd_waves(int mask_id, int D, int dtype, int T) {
    if (dtype == CHILL_F32 || D > 128) return 4;
    if (CHILL_TUNE_FWD_WAVES) return CHILL_TUNE_FWD_WAVES;
    (void)mask_id;
    return (D <= 64 || T <= kFwdShortSequence) ? 4 : 8;
}
constexpr int fwd_streamed(int mask_id, int D, int dtype, int T) {
    if (dtype == CHILL_F32) return 32;
    if (D > 128) return 64;
    if (CHILL_TUNE_FWD_STREAMED) return CHILL_TUNE_FWD_STREAMED;
    return (fwd_waves(mask_id, D, dtype, T) == 8 && !CHILL_FWD_FAST) ? 128 : 64;
}
// LDS stages of the forward K/V ring: two for the 4-wave shape of 16-bit inputs (so that two
// workgroups fit a CU); otherwise three (one tile resident ahead, one in flight) when they fit in
// 144 KiB, else two.
constexpr int fwd_stages(int mask_id, int D, int dtype, int T) {
    const int streamed = fwd_streamed(mask_id, D, dtype, T);
    if (dtype != CHILL_F32 && D <= 128) {
        if (CHILL_TUNE_FWD_STAGES) return CHILL_TUNE_FWD_STAGES;
        // the fast forward keeps one tile resident ahead of the one in use: three stages (two workgroups of
        // four waves still share a CU at head dim 64), four for the 8-wave workgroup that owns its CU
        if (fwd_waves(mask_id, D, dtype, T) == 4) return (CHILL_FWD_FAST && D == 64) ? 3 : 2;
        if (CHILL_FWD_FAST) return 4;
    }
    return 3 * fwd_stage_bytes(streamed, D, dtype) <= 144 * 1024 ? 3 : 2;
}
// 16-bit inputs at head dim 256: fwd_regs_kernel (O^T in hand-managed accumulation registers).
constexpr bool fwd_uses_regs(int D, int dtype) { return dtype != CHILL_F32 && D == 256; }

// Forward launches far too small for the chip (fwd_small_kernel): a workgroup of four waves owns 32
// query rows and its waves split the keys.  Per wave LDS holds a 32-row K block, a 32-row V block and
// the wave's running max and row sum; rows of at most 512 bytes, so that four such areas fit.
// For 16-bit inputs it is taken while its grid of B * H * T / 32 tiles is about what the chip holds at once
// (measured against the ordinary forward, causal and full masks, T = 128 .. 16384, 1 .. 128 heads: with up to
// 256 tiles it wins everywhere, by 1.1x .. 1.5x; with 512 it still wins at head dim 128, where a block is more
// work, and under causal-like masks; with 1024 it loses or ties); fp32 much further up (fwd_small_max_tiles).
constexpr int kFwdSmallWaves = 4;
// (sequences of up to 16384 rows: with a head or two of such a sequence the ordinary kernels have a few dozen workgroups.
// Measured at T = 8192: fp32 causal B1 H2 D64 forward 633 -> 193 us, dQ 883 -> 244, dK/dV 1032 -> 332, full mask
// 645 -> 340, 908 -> 408, 1047 -> 597; fp32 causal B1 H4 T16384 forward 1318 -> 1224, dQ 2800 -> 1570; bf16 causal
// B1 H2 D128 forward 142 -> 89, dQ 153 -> 90, full mask 145 -> 125 and 156 -> 132; bf16 causal B1 H1 D64 dQ 108 -> 54,
// dK/dV 110 -> 76)
constexpr int kFwdSmallMaxT = 16384;
// (at the end the area also takes the wave's partial O^T, 4 KiB per 32 columns of the head dim)
constexpr int fwd_small_wave_bytes(int D, int dtype) {
    const int blocks = 2 * 32 * D * elem_bytes(dtype), partial = ((D + 31) / 32) * 16 * 64 * 4;
    return (blocks > partial ? blocks : partial) + 2 * 64 * 4;
}
constexpr int fwd_small_lds_bytes(int D, int dtype) { return kFwdSmallWaves * fwd_small_wave_bytes(D, dtype); }
// fp32, whose ordinary kernels give a wave 32 rows and all their keys at 2 us and more per block, is served much
// further up since the small kernels balance their launches (small_takes_two_tiles, below).  Measured against
// fwd_kernel / dq_kernel / dkdv_kernel at head dims 32, 64 and 128, T = 512 .. 4096, 1536 .. 32768 tiles: under
// masks whose rows grow with their index (causal, prefix-LM) the forward wins up to 2048 tiles (B1 H24 T2048 D64:
// 300 -> 154 us; at 2048 tiles 373 -> 359, at 4096 +5 .. +9 %; head dim 128: 387 -> 317 at 1536 tiles, +11 .. +15 %
// at 2048), dQ up to 16384 tiles (8192 at head dim 128; B1 H24 T2048: 406 -> 195 us; B4 H16 T4096: 2000 -> 1750; head dim 128: 3925 -> 3820),
// dK/dV up to 4096 tiles at T <= 2048 (B4 H16 T2048: 797 -> 715 us; prefix-LM B8 H32 T1024, 8192 tiles: +9 %) and 1024
// at T = 4096 (B1 H8: 523 -> 333 us; B1 H16: 606 -> 645); under the other masks, whose tiles are all alike, forward
// and dQ win up to 1536 tiles (full mask B1 H24 T2048 D64: 318 -> 276 and 421 -> 337 us; sliding window 70 -> 60 and
// 104 -> 85) and tie or lose from 2048 on, and dK/dV does not win beyond its 512.
constexpr bool mask_rows_grow(int mask_id) { return mask_id == CHILL_MASK_CAUSAL || mask_id == CHILL_MASK_PREFIX_LM; }
constexpr long long fwd_small_max_tiles(int mask_id, int D, int dtype) {
    // (16-bit head dims <= 64 at 512 tiles: causal B1 H2 T8192 69 -> 57 us, B1 H4 T4096 38 -> 31; full mask 71 -> 81, 39 -> 42)
    if (dtype != CHILL_F32) return ((D >= 128 || mask_rows_grow(mask_id)) ? 2 : 1) * kComputeUnits;
    return (mask_rows_grow(mask_id) && D <= 64 ? 8 : 6) * kComputeUnits;
}
constexpr bool fwd_takes_small(int mask_id, long long batch_heads, int T, int D, int dtype) {
    return CHILL_TUNE_FWD_SMALL && D * elem_bytes(dtype) <= 512 && T <= kFwdSmallMaxT &&
           batch_heads * ((T + 31) / 32) <= fwd_small_max_tiles(mask_id, D, dtype);
}

// With more 32-row tiles than the chip has CUs the workgroups of a launch no longer run all at once or alone on their
// CUs, and under causal-like masks, where a tile's work grows with its index, the launch ends when the CU with the
// longest tiles does.  Then, in the forward and dQ, a workgroup of eight waves takes two tiles side by side, tile j
// from the end and tile j from the start of a head, which add up to the same work for every workgroup, where two areas
// fit in LDS (the wave then has 256 registers: enough for the forward and dQ, not for dK/dV with K, V and two
// accumulators); and every small launch takes its tiles longest first across all heads.  Measured on fp32 at head dim
// 64, forward / dQ / dK/dV: prefix-LM B1 H8 T2048 83 / 127 / 161 -> 66 / 87 / 127 us, causal 81 / 126 / 159 ->
// 52 / 69 / 97, causal B2 H8 T1024 45 / 71 / 90 -> 30 / 40 / 58; two tiles per workgroup against the new order
// alone: forward 66 against 69, dQ 87 against 101 us on the prefix-LM shape.
constexpr bool small_fits_two_tiles(int lds_bytes_one) { return 2 * lds_bytes_one <= 160 * 1024; }
constexpr bool small_takes_two_tiles(long long tiles) { return tiles > kComputeUnits; }
// what the report says of such a launch: 32 rows and 4 waves per tile; the LDS of the workgroup (of both tiles)
constexpr TileConfig small_tile_config(int lds_bytes_one, long long tiles) {
    return TileConfig{32, 32, kFwdSmallWaves,
                      (small_fits_two_tiles(lds_bytes_one) && small_takes_two_tiles(tiles)) ? 2 * lds_bytes_one : lds_bytes_one};
}

// The backward of such launches (dq_small_kernel, dkdv_small_kernel): the same split of the streamed
// axis over four waves; a wave's area holds two 32-row blocks (K and V, or Q and dO), later its partial
// accumulators (`outputs` x 4 KiB per 32 columns of the head dim), and LSE2 / delta of a query block.
#ifndef CHILL_TUNE_BWD_SMALL
#define CHILL_TUNE_BWD_SMALL 1
#endif
constexpr int bwd_small_wave_bytes(int D, int dtype, int outputs) {
    const int blocks = 2 * 32 * D * elem_bytes(dtype), partial = outputs * ((D + 31) / 32) * 16 * 64 * 4;
    return (blocks > partial ? blocks : partial) + 2 * 32 * 4;
}
constexpr int bwd_small_lds_bytes(int D, int dtype, int outputs) { return kFwdSmallWaves * bwd_small_wave_bytes(D, dtype, outputs); }
#ifndef CHILL_TUNE_BWD_SMALL_SCALE
#define CHILL_TUNE_BWD_SMALL_SCALE 1
#endif
// Where they win (measured against dq_kernel / dkdv_kernel on causal masks, 1 .. 128 heads, T = 128 .. 4096):
// dQ while its grid of B * H * T / 32 workgroups is at most 512 (256 for 16-bit inputs at head dim 128):
// 1.1x .. 1.9x for 16-bit inputs, 1.5x .. 3.8x for fp32; dK/dV at head dims up to 64 with at most 256 workgroups
// (512 for fp32): 1.1x .. 1.4x and 1.2x .. 3.4x.  At head dim 128 dK/dV does not win (a wave then holds K, V and
// two accumulators of 64 registers each), and fp32 rows of 512 bytes do not fit a wave's registers at all.
constexpr bool bwd_small_serves(int D, int dtype, int pass) {
    return CHILL_TUNE_BWD_SMALL && (pass == CHILL_PASS_DKDV ? D <= 64 : (D <= 128 && D * elem_bytes(dtype) <= 512));
}
// (fp32 beyond that: the measurements at fwd_small_max_tiles)
constexpr long long bwd_small_max_tiles(int mask_id, int T, int D, int dtype, int pass) {
    // (16-bit dQ at 512 tiles, head dim 128: causal B1 H2 T8192 153 -> 90 us, B1 H4 T4096 82 -> 50, B1 H16 T1024 27 -> 23, full
    // mask 156 -> 132 and 95 -> 75; at 1024 tiles wins and losses of up to 25 % either way)
    // (16-bit dK/dV at 512 tiles, head dim 64, causal: B1 H2 T8192 118 -> 90 us, B1 H4 T4096 62 -> 52, B1 H16 T1024 20 -> 22; full
    // mask 134 -> 164 and 76 -> 91)
    if (dtype != CHILL_F32) return ((pass == CHILL_PASS_DQ || (mask_rows_grow(mask_id) && T >= 4096)) ? 2 : 1) * kComputeUnits;
    // (dQ at 16384 tiles, causal B8 H16 T4096: head dim 64 3775 -> 3393 us, 32 2045 -> 1901, 128 7822 -> 7909; at 32768 +1 .. +14 %)
    if (pass == CHILL_PASS_DQ) return (mask_rows_grow(mask_id) ? (D <= 64 ? 64 : 32) : 6) * kComputeUnits;
    return (mask_rows_grow(mask_id) ? (T <= 2048 ? 16 : 4) : 2) * kComputeUnits;
}
constexpr bool bwd_takes_small(int mask_id, long long batch_heads, int T, int D, int dtype, int pass) {
    return bwd_small_serves(D, dtype, pass) && T <= kFwdSmallMaxT * CHILL_TUNE_BWD_SMALL_SCALE &&
           batch_heads * ((T + 31) / 32) <= bwd_small_max_tiles(mask_id, T, D, dtype, pass) * CHILL_TUNE_BWD_SMALL_SCALE;
}

constexpr TileConfig fwd_tile_config(int mask_id, int D, int dtype, int T = kLongSequence) {
    const int waves = fwd_waves(mask_id, D, dtype, T);
    const int streamed = fwd_streamed(mask_id, D, dtype, T);
    return TileConfig{waves * 32, streamed, waves,
                      fwd_stages(mask_id, D, dtype, T) * fwd_stage_bytes(streamed, D, dtype)};
}

// dQ.  16-bit inputs at head dim 128: 8 waves x 64 streamed keys in three stages; banded masks, head
// dims <= 64 and sequences up to kDqShortSequence: 4 waves x 64 keys in two stages, two workgroups per
// CU (prefix-LM at D = 64: dQ -9 %).  16-bit inputs at head dim 256: dq_regs_kernel (hand-managed
// accumulation registers), 4 waves, dq_regs_keys streamed keys per tile (0: the shape is served by
// dq_kernel).
constexpr int dq_regs_keys(int D, int dtype) { return (dtype != CHILL_F32 && D == 256) ? 32 : 0; }
constexpr int dq_waves(int mask_id, int D, int dtype, int T) {
    if (dtype == CHILL_F32 || D > 128) return 4;
    if (CHILL_TUNE_DQ_WAVES) return CHILL_TUNE_DQ_WAVES;
    return (mask_is_banded(mask_id) || D <= 64 || T <= kDqShortSequence) ? 4 : 8;
}
constexpr int dq_streamed(int D, int dtype) {
    if (dtype == CHILL_F32) return 32;
    if (D > 128) return dq_regs_keys(D, dtype) > 0 ? dq_regs_keys(D, dtype) : 32;
    return CHILL_TUNE_DQ_STREAMED ? CHILL_TUNE_DQ_STREAMED : 64;
}
// dQ LDS stage: swizzled (unpadded) K and V tiles.  Two stages for the 4-wave shape of 16-bit inputs;
// otherwise three when they fit in 144 KiB.
constexpr int dq_stages(int mask_id, int D, int dtype, int T) {
    if (dtype != CHILL_F32 && D <= 128) {
        if (CHILL_TUNE_DQ_STAGES) return CHILL_TUNE_DQ_STAGES;
        if (dq_waves(mask_id, D, dtype, T) == 4) return 2;
    }
    return 3 * 2 * dq_streamed(D, dtype) * D * elem_bytes(dtype) <= 144 * 1024 ? 3 : 2;
}

// 16-bit inputs at head dim 128 have a second dQ kernel (dq_regs2_kernel): 4 waves, one per SIMD, 64 query rows each
// with Q and dO in registers, 32-key tiles in four stages, runs of predicate-free tiles in a generated loop
// (gen_dq_loop.py).  It owns its CU; taken like its dK/dV counterpart for long sequences on grids of at least two
// workgroups per CU, not for the banded masks.  Measured on dQ alone, against dq_kernel on one box: causal B8 H16
// T8192 2.71 / 2.90 ms, B2 H8 T8192 0.408 / 0.428, prefix-LM B4 H16 T8192 1.45 / 1.55, full mask fp16 B4 H16 T4096
// 0.76 / 0.82; but causal B16 H16 T4096 1.63 / 1.62, B8 H8 T4096 0.509 / 0.496, B1 H8 T8192 0.227 / 0.232.
// (from 4097 keys on, where dq_kernel leaves its 4-wave shape; full masks from 2048.  Measured on bf16 at B8 H16 since
// the waves at a ragged end of the sequence take the complete tile's predicate-free range: causal T = 5000 / 6143 /
// 7000 / 8000 -7.7 / -8.1 / -4.9 / -5.3 %, at T = 4096 / 3072 / 2048 against the 4-wave shape +2 / +3 / +14 %; full mask
// T = 2048 / 3072 / 4096 / 6143 / 8000 -4 / -7 / -7 / -9.5 / -9.6 %; prefix-LM T = 5000 / 7000 -6.4 %, T = 3072 +0.5 %)
constexpr int dq_regs2_min_sequence(int mask_id) { return mask_id == CHILL_MASK_FULL ? 2048 : 4097; }
constexpr int kDqRegs2MinWorkgroups = 2 * 256;
constexpr bool dq_regs2_is_optional(int D, int dtype) { return dtype != CHILL_F32 && D == 128; }
constexpr bool dq_takes_regs2(int mask_id, long long batch_heads, int T) {
    return !mask_is_banded(mask_id) && T >= dq_regs2_min_sequence(mask_id) && batch_heads * ((T + 255) / 256) >= kDqRegs2MinWorkgroups;
}
constexpr TileConfig dq_regs2_tile_config(int D, int dtype) {
    return TileConfig{256, 32, 4, 4 * 2 * 32 * D * elem_bytes(dtype)};
}

// fp32 at head dim 256 (dq_split_kernel): two waves share a 32-query block; two stages of 32-key K and V
// tiles, then one 4 KiB slot per wave for the two products of a block.
constexpr bool dq_is_split(int D, int dtype) { return dtype == CHILL_F32 && D == 256; }
constexpr TileConfig dq_tile_config(int mask_id, int D, int dtype, int T = kLongSequence) {
    const int waves = dq_waves(mask_id, D, dtype, T);
    const int streamed = dq_streamed(D, dtype);
    if (dq_is_split(D, dtype)) return TileConfig{waves * 16, 32, waves, 2 * 2 * 32 * D * 4 + waves * 16 * 64 * 4};
    return TileConfig{waves * 32, streamed, waves,
                      dq_stages(mask_id, D, dtype, T) * 2 * streamed * D * elem_bytes(dtype)};
}

// dK/dV, rows of at most 256 bytes ("paired" kernel): a workgroup of 8 waves owns 128 key rows;
// pairs of waves share a 32-key block and split the streamed 64-row query tiles.  LDS: the resident
// K and V tiles plus two ring stages of swizzled Q and dO tiles with the LSE2 and delta of their rows.
// Longer rows: dkdv_split_kernel, below.
constexpr bool dkdv_is_paired(int D, int dtype) { return D * elem_bytes(dtype) <= 256; }
// 16-bit head dims <= 64: workgroups of 4 waves (64 key rows), small enough in LDS (50 KiB at D = 64)
// and registers (167) for two or three of them per CU, which hide each other's start and end
// (measured: sliding window dK/dV -32 %, prefix-LM at D = 64 -17 %).  At D = 128 the two-stage ring of
// such a workgroup takes 99 KiB; with a one-stage ring it fits twice but runs 8 % slower than the
// 8-wave workgroup.
// `small_grid`: the 8-wave grid would cover at most half of the CUs (dkdv_takes_small_row); then the
// 64-row workgroup is taken at every 16-bit head dim (B1 H8 T2048 D128: -17 %).
constexpr int dkdv_paired_waves(int mask_id, int D, int dtype, bool small_grid = false) {
    (void)mask_id;
    if (CHILL_TUNE_DKDV_WAVES) return CHILL_TUNE_DKDV_WAVES;
    return (dtype != CHILL_F32 && (D <= 64 || small_grid)) ? 4 : 8;
}
constexpr bool dkdv_takes_small_row(long long batch_kv_heads, int T) {
    return batch_kv_heads * ((T + 127) / 128) <= kComputeUnits / 2;
}
// at the end the waves of a pair exchange one fp32 accumulator each through LDS: 8 waves x (D rounded
// up to 32) x 32 floats
constexpr int dkdv_paired_exchange_bytes(int D) { return 8 * ((D + 31) / 32) * 16 * 64 * 4; }
// Longer rows (fp32 at head dims 128 and 256, dkdv_split_kernel): dkdv_split(D) waves share a 32-key
// block and its state; two ring stages of 32-row Q and dO tiles, then one 4 KiB slot per wave for the
// partial products.  Head dim 128: 8 waves, 128 key rows, two waves per SIMD; head dim 256: 4 waves
// on one 32-key block (two ring stages alone take 128 KiB).
constexpr int dkdv_split(int D) { return D >= 256 ? 4 : 2; }
constexpr int dkdv_split_waves(int D) { return D >= 256 ? 4 : 8; }
constexpr int dkdv_split_stage_bytes(int D, int dtype) { return 2 * 32 * D * elem_bytes(dtype) + 2 * 32 * 4; }
constexpr int dkdv_split_lds_bytes(int D, int dtype) {
    return 2 * dkdv_split_stage_bytes(D, dtype) + dkdv_split_waves(D) * 16 * 64 * 4;
}

// dK/dV with hand-managed accumulation registers (dkdv_regs_kernel, 16-bit inputs): 4 waves, K in
// registers, V in LDS, 32-row Q / dO tiles in a ring.  blocks = 32-key blocks per wave:
//   * head dim 256: one block per wave (128 key rows per workgroup), two ring stages: the only
//     kernel of that shape;
//   * head dims 64 and 128: two blocks per wave (256 key rows), four stages, beside the paired kernel
//     (dkdv_regs_is_optional below).
constexpr int dkdv_regs_blocks(int D, int dtype) {
    if (dtype == CHILL_F32) return 0;
    if (D == 256) return 1;
    return 0;
}
constexpr int dkdv_regs_stages(int D) { return D == 256 ? 2 : 4; }
// 16-bit inputs at head dims 64 and 128 have both kernels: the paired one, and dkdv_regs_kernel with two blocks per wave,
// whose runs of predicate-free tiles go through a generated loop (gen_bwd_loop.py).  The latter owns its CU (130 KiB of
// LDS, 512 registers per wave) and pays more before and after its loop (K into registers, V negated in LDS, no second
// workgroup to hide behind): it is taken for long sequences on a grid of at least two workgroups per CU, and of
// the banded masks only for those named below.  Measured on dK/dV alone, against the paired kernel:
// causal B8 H16 T8192 3.63 / 4.06 ms, B16 H16 T4096 2.18 / 2.27, B2 H8 T8192 0.547 / 0.591, full mask fp16 B4 H16
// T4096 0.98 / 1.16, prefix-LM B4 H16 T8192 1.91 / 2.16; but causal B1 H8 T8192 0.368 / 0.318, B4 H16 T2048
// 0.227 / 0.197, sliding window 512 at T8192 0.65 / 0.49.  At head dim 64 (against the 4-wave kernel that runs three
// to a CU): causal B8 H16 T4096 0.73 / 0.77, B4 H32 T8192 2.12 / 2.42, B2 H8 T8192 0.31 / 0.36, B1 H32 T16384 1.99 / 2.35,
// full mask B4 H16 T4096 0.56 / 0.73, prefix-LM B4 H32 T8192 2.12 / 2.45; there the other kernel's workgroups are a
// quarter of the size and fill a small grid better: B2 H16 T4096 (512 workgroups of this kernel) causal 0.20 / 0.17,
// prefix-LM 0.20 / 0.18 (but full mask 0.28 / 0.38); B4 H16 T4096 (1024) causal 0.37 / 0.38: from four workgroups per CU on.
constexpr int kDkdvRegsBlocks128 = 2;
// Sequence lengths from which it is taken, by what the mask leaves of a key block's loop (measured against the other
// kernel on bf16 grids of 1024 .. 4096 workgroups, B8 .. B32 H16): under a full mask every tile is predicate-free and it
// wins from the shortest sequences tried (T = 1024 / 2048 / 3072 / 4000: -16 / -17 / -18 / -17 % at head dim 128, -21 / -27 /
// -27 / -23 % at head dim 64); under a causal mask the first tiles of a key block run outside the generated loop and the
// runs shrink with the sequence (head dim 128: T = 1024 / 2048 / 3072 / 3500 / 4000 +14 / +1 / -3 / -4.5 / -5 .. -8 %;
// head dim 64: T = 2048 / 3072 / 3500 / 4000 +5 .. +17 / -2 .. +1.5 / -5 / -3 .. -5 %); prefix-LM lies between the two
// (prefix 512, head dim 128: -6 .. -10 % from T = 1024 on) and takes the causal limits; the banded masks it serves keep 4096.
constexpr int dkdv_regs_min_sequence(int mask_id, int D) {
    return mask_id == CHILL_MASK_FULL ? 1024 : mask_is_banded(mask_id) ? 4096 : D >= 128 ? 3072 : 3500;
}
constexpr int kDkdvRegsMinWorkgroups = 2 * 256;
constexpr int kDkdvRegsMinWorkgroups64 = 4 * 256;
// (by mask as well: under a full mask it wins on one workgroup per CU already, B1 H16 T4096 -24 % at head dim 128 and -38 %
// at head dim 64, where causal and prefix-LM masks lose 10-19 %; at head dim 64 the causal-like masks win on 512 workgroups
// from 8192 keys on, B1 H16 T8192 -13 %, B1 H8 T16384 -15 %, and lose 4-9 % at T = 4096)
constexpr long long dkdv_regs_min_workgroups(int mask_id, int D, int T) {
    if (mask_id == CHILL_MASK_FULL) return 256;
    if (D >= 128) return kDkdvRegsMinWorkgroups;
    return (!mask_is_banded(mask_id) && T >= 8192) ? kDkdvRegsMinWorkgroups64 / 2 : kDkdvRegsMinWorkgroups64;
}
constexpr bool dkdv_regs_is_optional(int D, int dtype) { return dtype != CHILL_F32 && (D == 128 || D == 64); }
// Banded masks take it only when a wave's 64 key rows lie in one chunk, so that its tiles are all predicate-free
// and all alike: chunkwise masks whose chunk size is a multiple of 64 (`mask_arg0` = the mask's first argument;
// measured at head dim 128, T = 8192 and 16384: chunks of 64 / 128 / 256 / 1024 rows -5 / -8 / -13 / -16 %, chunks
// of 96 rows +13 %; at head dim 64, where a tile is half the work, chunks of 64 rows +30 .. +68 %, of 128 rows +-1 %,
// of 256 rows 0 .. +8 %, of 320 rows -8 %, of 512 rows -19 %, of 1024 rows -17 %: from 320 rows on); and sliding
// windows from kDkdvRegsWideBand keys on (`band_keys` = mask_band_keys; windows of 64 .. 512 keys +32 .. +60 %,
// of 1024 +14 %, of 2048 -2 %, of 4096 -8 % at head dim 128 and -11 % at head dim 64).
constexpr int kDkdvRegsWideBand = 4096;
constexpr bool dkdv_regs_serves_band(int mask_id, long long mask_arg0, long long band_keys, int D) {
    return (mask_id == CHILL_MASK_CHUNKWISE && mask_arg0 % (32 * kDkdvRegsBlocks128) == 0 && (D >= 128 || mask_arg0 >= 320)) ||
           (mask_id == CHILL_MASK_SLIDING_WINDOW && band_keys >= kDkdvRegsWideBand);
}
constexpr bool dkdv_takes_regs(int mask_id, long long mask_arg0, long long band_keys, int D, long long batch_kv_heads, int T) {
    return (!mask_is_banded(mask_id) || dkdv_regs_serves_band(mask_id, mask_arg0, band_keys, D)) && T >= dkdv_regs_min_sequence(mask_id, D) &&
           batch_kv_heads * ((T + 128 * kDkdvRegsBlocks128 - 1) / (128 * kDkdvRegsBlocks128)) >= dkdv_regs_min_workgroups(mask_id, D, T);
}

// `regs`: the row of dkdv_regs_kernel where that kernel is an option (dkdv_regs_is_optional)
constexpr TileConfig dkdv_tile_config(int mask_id, int D, int dtype, bool small_grid = false, bool regs = false) {
    const int row_bytes = D * elem_bytes(dtype);
    const int blocks = (regs && dkdv_regs_is_optional(D, dtype)) ? kDkdvRegsBlocks128 : dkdv_regs_blocks(D, dtype);
    if (blocks > 0) {
        const int rows = 4 * 32 * blocks;
        return TileConfig{rows, 32, 4, rows * row_bytes + dkdv_regs_stages(D) * (2 * 32 * row_bytes + 2 * 32 * 4)};
    }
    if (dkdv_is_paired(D, dtype)) {
        const int waves = dkdv_paired_waves(mask_id, D, dtype, small_grid);
        const int rows = 16 * waves;
        const int ring = 2 * rows * row_bytes + 2 * (2 * 64 * row_bytes + 2 * 64 * 4);
        const int exchange = dkdv_paired_exchange_bytes(D) * waves / 8;
        return TileConfig{rows, 64, waves, ring > exchange ? ring : exchange};
    }
    return TileConfig{32 * dkdv_split_waves(D) / dkdv_split(D), 32, dkdv_split_waves(D), dkdv_split_lds_bytes(D, dtype)};
}

// batch_heads = B * H and T = sequence length of the launch (the forward and dQ rows depend on them);
// T = kLongSequence for the row of long sequences on a full chip.
// mask_arg0 = the mask's first argument (the dK/dV row of chunkwise masks depends on the chunk size), band_keys =
// mask_band_keys of the mask (the forward and dK/dV rows of banded masks depend on the width of the band).
inline int tile_config(int mask_id, long long mask_arg0, long long band_keys, int D, int dtype, int pass, long long batch_heads,
                       int T, TileConfig* out) {
    if (dtype != CHILL_F32 && dtype != CHILL_F16 && dtype != CHILL_BF16) return CHILL_ERR_BAD_DTYPE;
    if (D != 16 && D != 32 && D != 64 && D != 128 && D != 256) return CHILL_ERR_BAD_HEAD_DIM;
    switch (pass) {
        case CHILL_PASS_FWD:
            if (T != kLongSequence && fwd_takes_small(mask_id, batch_heads, T, D, dtype)) {
                *out = small_tile_config(fwd_small_lds_bytes(D, dtype), batch_heads * ((T + 31) / 32));
                return CHILL_OK;
            }
            *out = fwd_tile_config(mask_id, D, dtype, fwd_takes_short_row(mask_id, band_keys, batch_heads, T) ? 1 : kLongSequence);
            return CHILL_OK;
        case CHILL_PASS_DQ:
            if (T != kLongSequence && bwd_takes_small(mask_id, batch_heads, T, D, dtype, CHILL_PASS_DQ)) {
                *out = small_tile_config(bwd_small_lds_bytes(D, dtype, 1), batch_heads * ((T + 31) / 32));
                return CHILL_OK;
            }
            if (dq_regs2_is_optional(D, dtype) && (T == kLongSequence ? !mask_is_banded(mask_id) : dq_takes_regs2(mask_id, batch_heads, T))) {
                *out = dq_regs2_tile_config(D, dtype);
                return CHILL_OK;
            }
            *out = dq_tile_config(mask_id, D, dtype, (T != kLongSequence && dq_takes_short_row(batch_heads, T)) ? 1 : kLongSequence);
            return CHILL_OK;
        case CHILL_PASS_DKDV:
            // (for this pass batch_heads counts the key / value heads)
            if (T != kLongSequence && bwd_takes_small(mask_id, batch_heads, T, D, dtype, CHILL_PASS_DKDV)) {
                *out = TileConfig{32, 32, kFwdSmallWaves, bwd_small_lds_bytes(D, dtype, 2)};
                return CHILL_OK;
            }
            // (the row of long sequences on a full chip: the generated loop where there is one)
            *out = dkdv_tile_config(mask_id, D, dtype, T != kLongSequence && dkdv_takes_small_row(batch_heads, T),
                                    T == kLongSequence ? (!mask_is_banded(mask_id) || dkdv_regs_serves_band(mask_id, mask_arg0, band_keys, D))
                                                       : dkdv_takes_regs(mask_id, mask_arg0, band_keys, D, batch_heads, T));
            return CHILL_OK;
        default: return CHILL_ERR_BAD_ARGUMENT;
    }
}

// Work-item order: workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so the
// linear workgroup id is remapped to give every XCD a contiguous run of work items.  Returns the
// work item index or -1 when this workgroup has nothing to do.
//
// `resident` = workgroups of the kernel that share a CU.  A grid that the chip holds at once (more workgroups than CUs,
// at most `resident` per CU) is placed statically: the dispatcher deals an XCD's workgroups to its 32 CUs pass after
// pass in the same CU order, so workgroup l of an XCD and workgroup l + 32 share a CU.  The kernels order their
// work items longest first (under causal-like masks a tile's work grows with its index), which would hand a CU the
// longest items of both passes and another the shortest; every second pass is therefore taken in reverse, and the two
// items of a CU add up alike (measured on dq_kernel, 512 workgroups of four waves, causal bf16 at head dim 128:
// B1 H16 T4096 148 -> 113 us, B1 H32 T2048 82 -> 66, B2 H8 T4096 147 -> 116, B1 H8 T8192 216 -> 204).  Larger grids
// are dealt out as CUs become free, and longest first is the right order for that.
CHILL_HD int xcd_contiguous_item(int wg, int total, int resident = 1) {
    constexpr int kXcds = 8, kCusPerXcd = 32;
    const int per = (total + kXcds - 1) / kXcds;
    const int first = (wg % kXcds) * per;
    int local = wg / kXcds;
    if (resident > 1 && total > kXcds * kCusPerXcd && total <= resident * kXcds * kCusPerXcd) {
        const int pass = local / kCusPerXcd;
        if (pass & 1) {
            const int valid = total - first < per ? total - first : per;  // items of this XCD
            const int len = valid - pass * kCusPerXcd < kCusPerXcd ? valid - pass * kCusPerXcd : kCusPerXcd;
            const int c = local - pass * kCusPerXcd;
            if (c < len) local = pass * kCusPerXcd + len - 1 - c;
        }
    }
    const int item = first + local;
    return (local < per && item < total) ? item : -1;
}

}  // namespace chill
