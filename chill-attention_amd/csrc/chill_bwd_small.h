// dQ and dK/dV for launches too small to fill the chip: the streamed axis of a 32-row tile is split
// over the waves of its workgroup, as fwd_small_kernel does for the forward.
//
// dq_kernel gives a wave 32 query rows and all their keys, dkdv_kernel a pair of waves 32 keys and all
// their queries: with a handful of workgroups the run time is the longest row (or column), block after
// block.  Here a workgroup owns one 32-row block and its four waves take the 32-row blocks of the other
// axis in turn (wave w the blocks w, w + 4, ...), each with accumulators of its own, which are added up
// through LDS at the end (the gradients are sums over the streamed axis: chill_bwd_dq.py:303-332,
// chill_bwd_dkdv.py:366-410).  Every wave stages its blocks in an LDS area of its own, so the loops need
// no workgroup barrier.
#pragma once

#include "chill_device.h"
#include "chill_mask.h"
#include "chill_params.h"
#include "chill_tiles.h"

namespace chill {

// Adds up the waves' partial accumulators (NB blocks of 16 registers per lane, staged at `area` of every
// wave: register r of block i of lane l at ((i * 16 + r) * 64 + l) * 4) and stores this wave's share of
// the finished row blocks: lane (n, h) holds, of row n, the columns 32 * db + 8 * (r / 4) + 4 * h + r % 4.
// Block i of the accumulators goes to out[i / DB] (dQ: one output; dK/dV: two).
template <typename E, int D, int NOUT>
__device__ __forceinline__ void bwd_small_merge(const char* smem, int wave_bytes, int wave, int lane,
                                                typename Elem<E>::type* const (&row)[NOUT], const float (&mult)[NOUT],
                                                bool in_tensor, bool valid) {
    using ET = typename Elem<E>::type;
    constexpr int NW = kFwdSmallWaves;
    constexpr int DB = (D + 31) / 32;
    const int h = lane >> 5;
    if (!in_tensor) return;
    for (int i = wave; i < NOUT * DB; i += NW) {
        const int o = i / DB, db = i % DB;
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < NW; w++) {
                const float* part = reinterpret_cast<const float*>(smem + w * wave_bytes);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] += part[(i * 16 + 4 * g4 + e) * 64 + lane];
            }
            const int d0 = 32 * db + 8 * g4 + 4 * h;
            if (D >= 32 || d0 < D) {
#pragma unroll
                for (int e = 0; e < 4; e++) row[o][d0 + e] = (ET)(valid ? acc[e] * mult[o] : 0.f);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------ dQ
// TILES = 2: a workgroup of eight waves takes two 32-row blocks side by side, block j from the long end and block j
// from the short end of one head, four waves each with an LDS area of their own, as fwd_small_kernel does; the two
// halves meet at the one barrier of the kernel and nowhere else.
template <typename E, int D, int MASK, int TILES>
__global__ __launch_bounds__(kFwdSmallWaves * 64 * TILES) void dq_small_kernel(BwdParams p, int n_q_tiles, int total_items,
                                                                               int has_full_blocks) {
    using ET = typename Elem<E>::type;
    typedef LdsTile<E, D> L;
    constexpr int NW = kFwdSmallWaves;
    constexpr int NT = NW * 64;
    constexpr int DB = (D + 31) / 32;
    constexpr int TILE_BYTES = L::bytes(32);
    constexpr int WAVE_BYTES = bwd_small_wave_bytes(D, Elem<E>::kDType, 1);
    extern __shared__ __attribute__((aligned(16))) char smem_all[];

    const int item = blockIdx.x;
    if (item >= total_items) return;
    const int half = TILES == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / NT) : 0;  // which block of the workgroup
    char* smem = smem_all + half * (NW * WAVE_BYTES);
    // the blocks of all heads from the long end to the short end (under causal-like masks: longest first, so that a launch
    // of more workgroups than fit at once ends without stragglers); pairs of blocks: all of the same length
    const int per_head = TILES == 2 ? (n_q_tiles + 1) / 2 : n_q_tiles;
    const int n_heads = total_items / per_head;
    const int bh = item % n_heads;
    const int j = item / n_heads;
    const int qt = half == 0 ? n_q_tiles - 1 - j : j;
    // (an odd number of blocks: the middle one has no partner)
    const bool has_tile = half == 0 || n_q_tiles - 1 - j != j;
    const int b = bh / p.H;
    const int hd = bh % p.H;
    const int hkv = hd / p.group;

    const int tid = threadIdx.x % NT;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    const int qb = qt * 32;
    ET* dqbase = reinterpret_cast<ET*>(p.dq) + b * p.sdq.b + hd * p.sdq.h;
    if (!has_tile || qb >= seq_len) {
        if (has_tile) {
            // rows at or beyond lens[b] receive 0 (the reference relies on the adapter's zero-fill, chill.py:292)
            zero_rows<E, D, NT>(dqbase, p.sdq.t, qb, imin(32, p.T - qb), tid);
            if (p.delta_out != nullptr) {
                // (the dK/dV launch that follows reads delta of every row of the tiles it visits)
                for (int i = tid; i < imin(32, p.T - qb); i += NT) p.delta_out[b * p.delta_b + hd * p.delta_h + qb + i] = 0.f;
            }
        }
        if constexpr (TILES == 2) __syncthreads();  // the other half's one barrier
        return;
    }

    const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h;
    const ET* doptr = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hd * p.sdo.h;
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;

    // the 32-key blocks of these rows (utils.py:221-272 with 32 x 32 tiles)
    const TileRange wr = tile_range<MASK, true>(qb, 32, 32, seq_len, has_full_blocks != 0, p.margs);

    char* mine = smem + wave * WAVE_BYTES;
    AsyncSwizzledLoader<E, D, 32, 64> load_k, load_v;
    load_k.init(p.sk.t, 0, lane);
    load_v.init(p.sv.t, 0, lane);
    auto issue_block = [&](int blk) {
        const int k0 = blk * 32;
        load_k.issue(kptr + (int64_t)k0 * p.sk.t, p.T - k0, mine, 0, lane);
        load_v.issue(vptr + (int64_t)k0 * p.sv.t, p.T - k0, mine + TILE_BYTES, 0, lane);
    };
    const int first = wr.start + wave;
    if (first < wr.end) issue_block(first);

    // Q and dO rows as resident B operands; LSE2 and delta of the lane's row
    Resident<E, D> qf, dof;
    load_resident<E, D>(qf, qptr + (int64_t)qb * p.sq.t, p.sq.t, p.T - qb, lane);
    load_resident<E, D>(dof, doptr + (int64_t)qb * p.sdo.t, p.sdo.t, p.T - qb, lane);
    const int q_pos = qb + n;
    float lse_q = 0.f, delta_q = 0.f;
    if (q_pos < p.T) lse_q = p.lse[b * p.lse_b + hd * p.lse_h + q_pos];
    if (p.delta_out != nullptr) {
        // (every wave of the workgroup holds the same 32 rows; the first one writes)
        const ET* optr = reinterpret_cast<const ET*>(p.o) + b * p.so.b + hd * p.so.h;
        delta_q = resident_row_delta<E, D>(dof, optr + (int64_t)qb * p.so.t, p.so.t, p.T - qb, lane);
        if (wave == 0 && (lane >> 5) == 0 && q_pos < p.T) p.delta_out[b * p.delta_b + hd * p.delta_h + q_pos] = delta_q;
    } else if (q_pos < p.T) {
        delta_q = p.delta[b * p.delta_b + hd * p.delta_h + q_pos];
    }
    OperandOffsets<E, D> ofs;
    ofs.init(lane);

    f32x16 dq[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) dq[i][r] = 0.f;
    const lds_char* ktile = (const lds_char*)mine;
    const lds_char* vtile = ktile + TILE_BYTES;

    for (int blk = first; blk < wr.end; blk += NW) {
        wait_async_tiles();
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            s[r] = 0.f;
            dp[r] = 0.f;
        }
        // S^T and dP^T blocks: rows = keys 8 * (r / 4) + 4 * h + r % 4 of the block, column n = query row
        s = mma_rowwise<E, D>(ktile, 0, ofs, qf, s, lane);
        dp = mma_rowwise<E, D>(vtile, 0, ofs, dof, dp, lane);
        const bool full = blk >= wr.full_start && blk < wr.full_end;
        auto pos = [&](int r, int& q, int& k, float& lse, float& delta) {
            q = q_pos;
            k = blk * 32 + 8 * (r / 4) + 4 * h + (r % 4);
            lse = lse_q;
            delta = delta_q;
        };
        if (full)
            softmax_grad_block<MASK, false>(s, dp, p.scale_log2, seq_len, p.margs, pos);
        else
            softmax_grad_block<MASK, true>(s, dp, p.scale_log2, seq_len, p.margs, pos);
        mma_transposed<E, D>(ktile, 0, ofs, dp, dq, lane);  // dQ^T += K^T dS^T
        // the staging area is free once the MFMAs above have their operands
        if (blk + NW < wr.end) issue_block(blk + NW);
    }

    {
        float* my = reinterpret_cast<float*>(mine);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) my[(db * 16 + r) * 64 + lane] = dq[db][r];
    }
    __syncthreads();
    ET* const rows[1] = {dqbase + (int64_t)q_pos * p.sdq.t};
    const float mult[1] = {p.sm_scale};
    bwd_small_merge<E, D, 1>(smem, WAVE_BYTES, wave, lane, rows, mult, q_pos < p.T, q_pos < seq_len);
}

// ------------------------------------------------------------------------------------------ dK, dV
template <typename E, int D, int MASK>
__global__ __launch_bounds__(kFwdSmallWaves * 64) void dkdv_small_kernel(BwdParams p, int n_k_tiles, int total_items,
                                                                         int has_full_blocks) {
    using ET = typename Elem<E>::type;
    typedef LdsTile<E, D> L;
    constexpr int NW = kFwdSmallWaves;
    constexpr int NT = NW * 64;
    constexpr int DB = (D + 31) / 32;
    constexpr int TILE_BYTES = L::bytes(32);
    constexpr int WAVE_BYTES = bwd_small_wave_bytes(D, Elem<E>::kDType, 2);
    constexpr int VEC_OFF = WAVE_BYTES - 2 * 32 * 4;  // LSE2 and delta of the staged query rows
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int item = blockIdx.x;
    if (item >= total_items) return;
    // the key blocks of all heads from the first to the last (under causal-like masks: longest first, so that a launch of
    // more workgroups than fit at once ends without stragglers)
    const int n_heads = total_items / n_k_tiles;
    const int bh = item % n_heads;
    const int kt = item / n_heads;
    const int b = bh / p.H_kv;
    const int hkv = bh % p.H_kv;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    const int kb0 = kt * 32;
    ET* dkbase = reinterpret_cast<ET*>(p.dk) + b * p.sdk.b + hkv * p.sdk.h;
    ET* dvbase = reinterpret_cast<ET*>(p.dv) + b * p.sdv.b + hkv * p.sdv.h;
    if (kb0 >= seq_len) {
        // rows at or beyond lens[b] receive 0 (the reference relies on the adapter's zero-fill, chill.py:293-294)
        const int nrows = imin(32, p.T - kb0);
        zero_rows<E, D, NT>(dkbase, p.sdk.t, kb0, nrows, tid);
        zero_rows<E, D, NT>(dvbase, p.sdv.t, kb0, nrows, tid);
        return;
    }

    // the 32-query blocks that see these keys
    const TileRange wr = tile_range<MASK, false>(kb0, 32, 32, seq_len, has_full_blocks != 0, p.margs);
    const int n_blocks = wr.end - wr.start;
    const int n_iters = n_blocks * p.group;  // every query head of the GQA group in turn (chill_bwd_dkdv.py:156)

    char* mine = smem + wave * WAVE_BYTES;
    AsyncSwizzledLoader<E, D, 32, 64> load_q, load_do;
    load_q.init(p.sq.t, 0, lane);
    load_do.init(p.sdo.t, 0, lane);
    // iteration it = (group head, query block)
    auto issue_iter = [&](int it) {
        const int hq = hkv * p.group + it / n_blocks;
        const int q0 = (wr.start + it % n_blocks) * 32;
        const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hq * p.sq.h;
        const ET* doptr = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hq * p.sdo.h;
        load_q.issue(qptr + (int64_t)q0 * p.sq.t, p.T - q0, mine, 0, lane);
        load_do.issue(doptr + (int64_t)q0 * p.sdo.t, p.T - q0, mine + TILE_BYTES, 0, lane);
        // LSE2 (lanes 0..31) and delta (lanes 32..63) of the block's rows; rows past the end read as zero
        const int qq = q0 + n;
        const float* src = h == 0 ? p.lse + b * p.lse_b + hq * p.lse_h : p.delta + b * p.delta_b + hq * p.delta_h;
        reinterpret_cast<float*>(mine + VEC_OFF)[lane] = qq < p.T ? src[qq] : 0.f;
    };
    if (wave < n_iters) issue_iter(wave);

    // K and V rows as resident B operands
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;
    Resident<E, D> kf, vf;
    load_resident<E, D>(kf, kptr + (int64_t)kb0 * p.sk.t, p.sk.t, p.T - kb0, lane);
    load_resident<E, D>(vf, vptr + (int64_t)kb0 * p.sv.t, p.sv.t, p.T - kb0, lane);
    const int k_pos = kb0 + n;
    OperandOffsets<E, D> ofs;
    ofs.init(lane);

    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            dk[i][r] = 0.f;
            dv[i][r] = 0.f;
        }
    const lds_char* qtile = (const lds_char*)mine;
    const lds_char* dotile = qtile + TILE_BYTES;
    const lds_float* vec = reinterpret_cast<const lds_float*>(qtile + VEC_OFF);

    for (int it = wave; it < n_iters; it += NW) {
        wait_async_tiles();
        const int blk = wr.start + it % n_blocks;
        f32x4 lse4[4], del4[4];
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
            lse4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + 8 * g4 + 4 * h);
            del4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + 32 + 8 * g4 + 4 * h);
        }
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            s[r] = 0.f;
            dp[r] = 0.f;
        }
        // S and dP blocks: rows = queries 8 * (r / 4) + 4 * h + r % 4 of the block, column n = key
        s = mma_rowwise<E, D>(qtile, 0, ofs, kf, s, lane);
        dp = mma_rowwise<E, D>(dotile, 0, ofs, vf, dp, lane);
        const bool full = blk >= wr.full_start && blk < wr.full_end;
        auto pos = [&](int r, int& q, int& k, float& lse, float& delta) {
            q = blk * 32 + 8 * (r / 4) + 4 * h + (r % 4);
            k = k_pos;
            lse = lse4[r / 4][r % 4];
            delta = del4[r / 4][r % 4];
        };
        if (full)
            softmax_grad_block<MASK, false>(s, dp, p.scale_log2, seq_len, p.margs, pos);
        else
            softmax_grad_block<MASK, true>(s, dp, p.scale_log2, seq_len, p.margs, pos);
        mma_transposed<E, D>(dotile, 0, ofs, s, dv, lane);  // dV^T += dO^T P
        mma_transposed<E, D>(qtile, 0, ofs, dp, dk, lane);  // dK^T += Q^T dS
        // the staging area is free once the MFMAs above have their operands
        if (it + NW < n_iters) issue_iter(it + NW);
    }

    {
        float* my = reinterpret_cast<float*>(mine);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                my[(db * 16 + r) * 64 + lane] = dk[db][r];
                my[((DB + db) * 16 + r) * 64 + lane] = dv[db][r];
            }
    }
    __syncthreads();
    ET* const rows[2] = {dkbase + (int64_t)k_pos * p.sdk.t, dvbase + (int64_t)k_pos * p.sdv.t};
    const float mult[2] = {p.sm_scale, 1.f};
    bwd_small_merge<E, D, 2>(smem, WAVE_BYTES, wave, lane, rows, mult, k_pos < p.T, k_pos < seq_len);
}

}  // namespace chill
