// Forward for launches too small to fill the chip (a few heads of a short sequence): the keys of a
// q-tile are split over the waves of its workgroup.
//
// fwd_kernel gives a wave 32 query rows and all their keys; with B * H * T / 128 workgroups far below
// the number of CUs its run time is the length of the longest row, one 32-key block after the other
// (fp32, head dim 64: 2 us per block).  Here a workgroup owns 32 query rows only and its NW waves take
// the 32-key blocks of those rows in turn (wave w the blocks w, w + NW, ...), each with its own running
// max, row sum and O^T accumulator (chill_fwd.py:214-231, one wave's share of the keys); at the end the
// partial results are merged through LDS the way two halves of a softmax merge: everything is rescaled
// to the largest of the running maxima.  Every wave stages its K / V blocks in an LDS region of its
// own, so the loop needs no workgroup barrier.
#pragma once

#include "chill_device.h"
#include "chill_mask.h"
#include "chill_params.h"
#include "chill_tiles.h"

namespace chill {

// (kFwdSmallWaves, fwd_small_lds_bytes and the launches that come here: chill_tiles.h)

// TILES = 2: a workgroup of eight waves takes two q-tiles side by side, tile j from the end and tile j from the start of
// one head, four waves each with an LDS area of their own.  Under causal-like masks the two add up to the same work
// for every workgroup, where workgroups of one q-tile each leave the CUs that drew two long ones to finish alone
// (taken when the launch has more workgroups than the chip has CUs: fwd_small_tiles).  The two halves meet at the
// one barrier of the kernel and nowhere else.
template <typename E, int D, int MASK, int TILES>
__global__ __launch_bounds__(kFwdSmallWaves * 64 * TILES) void fwd_small_kernel(FwdParams p, int n_q_tiles, int total_items,
                                                                                int has_full_blocks) {
    using ET = typename Elem<E>::type;
    using M = Mask<MASK>;
    typedef LdsTile<E, D> L;
    constexpr int NW = kFwdSmallWaves;
    constexpr int NT = NW * 64;
    constexpr int DB = (D + 31) / 32;
    constexpr int TILE_BYTES = L::bytes(32);
    // K block, V block (later the partial O^T); then m and l of the wave's lanes
    constexpr int WAVE_BYTES = fwd_small_wave_bytes(D, Elem<E>::kDType);
    constexpr int ML_OFF = WAVE_BYTES - 2 * 64 * 4;
    extern __shared__ __attribute__((aligned(16))) char smem_all[];

    const int item = blockIdx.x;
    if (item >= total_items) return;
    const int half = TILES == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / NT) : 0;  // which q-tile of the workgroup
    char* smem = smem_all + half * (NW * WAVE_BYTES);
    // the q-tiles of all heads from the last to the first (under causal-like masks: longest first, so that a launch of
    // more workgroups than fit at once ends without stragglers); pairs of q-tiles: all of the same length
    const int per_head = TILES == 2 ? (n_q_tiles + 1) / 2 : n_q_tiles;
    const int n_heads = total_items / per_head;
    const int bh = item % n_heads;
    const int j = item / n_heads;
    const int qt = half == 0 ? n_q_tiles - 1 - j : j;
    // (an odd number of q-tiles: the middle one has no partner)
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
    ET* obase = reinterpret_cast<ET*>(p.o) + b * p.so.b + hd * p.so.h;
    float* lse_base = p.lse ? p.lse + b * p.lse_b + hd * p.lse_h : nullptr;
    if (!has_tile || qb >= seq_len) {
        if (has_tile) {
            // nothing attends here: the output rows are defined to be zero (chill.py:96, chill_fwd.py:70-71)
            const int nrows = imin(32, p.T - qb);
            zero_rows<E, D, NT>(obase, p.so.t, qb, nrows, tid);
            if (lse_base)
                for (int i = tid; i < nrows; i += NT) lse_base[qb + i] = 0.f;
        }
        if constexpr (TILES == 2) __syncthreads();  // the other half's one barrier
        return;
    }

    const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h;
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

    Resident<E, D> qf;
    load_resident<E, D>(qf, qptr + (int64_t)qb * p.sq.t, p.sq.t, p.T - qb, lane);
    OperandOffsets<E, D> ofs;
    ofs.init(lane);

    f32x16 o[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] = 0.f;
    float m_run = -INFINITY;  // running max of the row over this wave's keys (scaled, log2 domain)
    float l_run = 0.f;        // this lane's share of the row sum
    const int q_pos = qb + n;
    const float scale = p.scale_log2;
    const lds_char* ktile = (const lds_char*)mine;
    const lds_char* vtile = ktile + TILE_BYTES;

    for (int blk = first; blk < wr.end; blk += NW) {
        wait_async_tiles();
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
        // S^T block: rows = keys 8 * (r / 4) + 4 * h + r % 4 of the block, column n = query row
        s = mma_rowwise<E, D>(ktile, 0, ofs, qf, s, lane);
        const bool full = blk >= wr.full_start && blk < wr.full_end;
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float x = s[r] * scale;
            if (!full) {
                const int key = blk * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                const bool ok = (key < seq_len) && M::pred(q_pos, key, seq_len, p.margs);
                x = ok ? x : -INFINITY;
            }
            s[r] = x;
            mx = fmaxf(mx, x);
        }
        mx = max_across_halves(mx);
        // online softmax (chill_fwd.py:214-226); a row that has seen no key keeps 0 as its reference
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(((m_run == -INFINITY) ? 0.f : m_run) - m_use);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            s[r] = fast_exp2(s[r] - m_use);
            psum += s[r];
        }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        mma_transposed<E, D>(vtile, 0, ofs, s, o, lane);  // O^T += V^T P^T
        // the staging area is free once the MFMAs above have their operands
        if (blk + NW < wr.end) issue_block(blk + NW);
    }

    // ---- merge the waves' partial results
    // m and the row sum (both halves of a row added up) of every wave; then O^T of every wave over its
    // own staging area: register r of head-dim block db of lane l at ((db * 16 + r) * 64 + l) * 4
    const float l_row = sum_across_halves(l_run);
    float* my_ml = reinterpret_cast<float*>(mine + ML_OFF);
    my_ml[lane] = m_run;
    my_ml[64 + lane] = l_row;
    {
        float* my_o = reinterpret_cast<float*>(mine);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) my_o[(db * 16 + r) * 64 + lane] = o[db][r];
    }
    __syncthreads();
    float m_all = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; w++) m_all = fmaxf(m_all, reinterpret_cast<const float*>(smem + w * WAVE_BYTES + ML_OFF)[lane]);
    const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
    float weight[NW];
    float l_all = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
        const float* ml = reinterpret_cast<const float*>(smem + w * WAVE_BYTES + ML_OFF);
        const float mw = ml[lane];
        weight[w] = (mw == -INFINITY) ? 0.f : fast_exp2(mw - m_ref);
        l_all += ml[64 + lane] * weight[w];
    }
    const float l_safe = (l_all == 0.f) ? 1.f : l_all;
    const float inv = 1.f / l_safe;
    const bool valid = q_pos < seq_len;
    // wave w finishes the head-dim blocks w, w + NW, ...: lane (n, h) holds, of ITS row, the columns
    // d = 32 * db + 8 * (r / 4) + 4 * h + r % 4
    if (q_pos < p.T) {
        ET* orow = obase + (int64_t)q_pos * p.so.t;
        for (int db = wave; db < DB; db += NW) {
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < NW; w++) {
                    const float* wo = reinterpret_cast<const float*>(smem + w * WAVE_BYTES);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[e] += wo[(db * 16 + 4 * g4 + e) * 64 + lane] * weight[w];
                }
                const int d0 = 32 * db + 8 * g4 + 4 * h;
                if (D >= 32 || d0 < D) {
#pragma unroll
                    for (int e = 0; e < 4; e++) orow[d0 + e] = (ET)(valid ? acc[e] * inv : 0.f);
                }
            }
        }
        // LSE2 = m + log2(l) (chill_fwd.py:288-289); -inf for a row that saw no key, 0 for rows past lens
        if (lse_base != nullptr && wave == 0 && h == 0) lse_base[q_pos] = valid ? m_all + __log2f(l_safe) : 0.f;
    }
}

}  // namespace chill
