// Forward kernel: O = softmax(mask(Q K^T * scale)) V and LSE2, one workgroup per (batch, head,
// q-tile) — the gfx950 counterpart of the reference's Triton program _chill_attn_fwd
// (chill_attention/chill_fwd.py:21-359).
//
// Each wave owns 32 query rows.  It keeps Q^T as MFMA B operands in registers and computes the
// TRANSPOSED score block S^T = K Q^T, so that in the accumulator layout one lane holds scores of
// a single query row: the running max / sum of the online softmax (chill_fwd.py:214-226) are
// per-lane scalars, and the only cross-lane step is one v_permlane32_swap per block.  P^T in
// accumulator layout is directly the B operand of O^T += V^T P^T; V^T comes out of LDS through
// the transposing read (ds_read_b64_tr_b16), so V is staged in its natural row-major form.
//
// K/V tiles are staged by the whole workgroup through a ring of padded LDS stages filled by
// asynchronous global->LDS loads: while tile i is consumed, tile i+1 is already resident and
// tile i+2 is in flight.  Work proceeds in steps of 32 keys, software-pipelined: the score MFMAs of
// step t+1 are issued before the softmax of step t, so matrix and vector units overlap in a wave.
//
// The softmax rescales lazily.  fp32 inputs: a row's reference max is raised (and O, l rescaled) only
// when a block max exceeds it by more than kRescaleTau, a wave-uniform rare branch.  16-bit inputs
// compute no block max at all on the common path: a row keeps the max of its first visible block as
// reference while the block sums of P stay below a limit far inside the range of P's type (fp16:
// 2^15, bf16: 1e18), and only a block whose sum exceeds it (or a row without reference yet) takes the
// branch that computes the block max, raises the reference and redoes the block's P from the raw
// scores, which are kept until then (chill_fwd.py:213-222 recomputes the max for every block; O and
// LSE2 do not depend on the reference beyond rounding).
//
// Tile skipping and the predicate-free path follow chill_fwd.py:131-139 and :161-185, evaluated
// per WAVE (32 rows): a wave skips streamed tiles outside its own k-range and drops the predicate
// inside its own full range.  The workgroup stages the hull of its waves' ranges.
#pragma once

#include <type_traits>

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"

namespace chill {

// Lazy-rescale threshold of the online softmax, in log2 units: P stays below 2^kRescaleTau.
constexpr float kRescaleTau = 8.0f;

template <typename E, int D, int TK>
struct FwdLds {
    typedef PaddedTile<E, D, rowwise_pad<E, D>()> KT;
    typedef PaddedTile<E, D, transposed_pad<E, D>()> VT;
    static constexpr int K_BYTES = KT::bytes(TK);
    static constexpr int V_BYTES = VT::bytes(TK);
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
};

// One q-tile (TQ = 32 * NW query rows of one head) from start to finish.
template <typename E, int D, int MASK, int NW, int TK, int NS>
__device__ __forceinline__ void fwd_q_tile(const FwdParams& p, char* smem, int b, int hd, int qt,
                                           int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    using M = Mask<MASK>;
    typedef FwdLds<E, D, TK> Lds;
    typedef typename Lds::KT KT;
    typedef typename Lds::VT VT;
    constexpr int TQ = NW * 32;
    constexpr int NT = NW * 64;
    constexpr int KB = TK / 32;         // 32-key blocks ("steps") per streamed tile
    constexpr int DB = (D + 31) / 32;   // 32-wide blocks of the head dim
    constexpr int NJ = KT::CH / 2;      // 16-byte chunk pairs along the head dim
    constexpr int LA = NS - 2;          // tiles certified resident ahead of the one being consumed
    static_assert(NS == 2 || NS == 3, "two or three LDS stages");
    const int hkv = hd / p.group;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    const int qb = qt * TQ;
    ET* obase = reinterpret_cast<ET*>(p.o) + b * p.so.b + hd * p.so.h;
    float* lse_base = p.lse ? p.lse + b * p.lse_b + hd * p.lse_h : nullptr;

    if (qb >= seq_len) {
        // nothing attends here: the output rows are defined to be zero (chill.py:96, chill_fwd.py:70-71)
        int nrows = imin(TQ, p.T - qb);
        zero_rows<E, D, NT>(obase, p.so.t, qb, nrows, tid);
        if (lse_base)
            for (int i = tid; i < nrows; i += NT) lse_base[qb + i] = 0.f;
        return;
    }

    const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h;
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;

    const TileRange wg = tile_range<MASK, true>(qb, TQ, TK, seq_len, false, p.margs);
    const int n_tiles = wg.end - wg.start;
    AsyncPaddedLoader<E, D, rowwise_pad<E, D>(), TK, NT> load_k;
    AsyncPaddedLoader<E, D, transposed_pad<E, D>(), TK, NT> load_v;
    load_k.init(p.sk.t, wave, lane);
    load_v.init(p.sv.t, wave, lane);
    auto issue_tile = [&](int i, int st_index) {
        int k0 = (wg.start + i) * TK;
        char* st = smem + st_index * Lds::STAGE_BYTES;
        load_k.issue(kptr + (int64_t)k0 * p.sk.t, p.sk.t, p.T - k0, st, wave, lane);
        load_v.issue(vptr + (int64_t)k0 * p.sv.t, p.sv.t, p.T - k0, st + Lds::K_BYTES, wave, lane);
    };
#pragma unroll
    for (int i = 0; i <= LA; i++)
        if (i < n_tiles) issue_tile(i, i);

    const int qw = qb + 32 * wave;
    Resident<E, D> qf;
    load_resident<E, D>(qf, qptr + (int64_t)qw * p.sq.t, p.sq.t, p.T - qw, lane);

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    if (qw < seq_len) wr = tile_range<MASK, true>(qw, 32, TK, seq_len, wave_has_full_blocks != 0, p.margs);
    // this wave's tiles, as offsets into the workgroup's ring
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    // per-lane LDS offsets inside a stage; everything else is an immediate
    const int k_lane = n * KT::PITCH + h * 16;
    int v_lane;
    if constexpr (Elem<E>::k16) {
        const int r = lane & 15, colgrp = (lane >> 4) & 1;
        int col = 16 * colgrp + 4 * (r & 3);
        if (D < 32) col &= (D - 1);
        v_lane = Lds::K_BYTES + (4 * h + (r >> 2)) * VT::PITCH + col * 2;
    } else {
        v_lane = Lds::K_BYTES + 4 * h * VT::PITCH + (D < 32 ? (n & (D - 1)) : n) * 4;
    }

    f32x16 o[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] = 0.f;
    float m_run = -INFINITY;  // reference max of the row (scaled, log2 domain)
    float m_use = 0.f;        // m_run, or 0 while the row has seen no unmasked key
    float l_run = 0.f;        // this lane's share of the row sum
    const int q_pos = qw + n;
    const Range vis = visible_range<MASK, true>(q_pos, seq_len, p.margs);  // the keys this lane's row sees
    // A negative scale reverses the order of the scores: the sign goes into Q, the softmax works
    // with |scale| (max(scale * s) = |scale| * max(sign * s)).
    const float scale = fabsf(p.scale_log2);
    // guarded softmax (16-bit inputs): see the step
    // not for the banded masks: their rows end after a few blocks, of which the first always takes the branch
    // (chunkwise fp16 T=16384 D=128: forward 0.43 ms with the guard, 0.42 without)
    constexpr bool kGuard = Elem<E>::k16 && !mask_is_banded(MASK);
    // a block sum below the limit keeps every P of the block inside fp16 (65504) / far inside bf16
    constexpr float kGuardLimit = Elem<E>::kDType == CHILL_F16 ? 32768.f : 1.0e18f;
    float guard_above = -1.f;

    // K operands of the score block of step kb of the tile at `stage` (rows 32*kb .. 32*kb+31),
    // read one step ahead of the MFMAs that consume them
    struct KOperands {
        i32x4 c[NJ];
    };
    auto load_k_operands = [&](KOperands& ko, const lds_char* stage, int kb) {
        const lds_char* base = stage + k_lane + kb * 32 * KT::PITCH;
#pragma unroll
        for (int j = 0; j < NJ; j++) ko.c[j] = *reinterpret_cast<const lds_i32x4*>(base + j * 32);
    };
    // S^T block: K[32 rows][:] Q^T
    auto scores = [&](f32x16& dst, const KOperands& ko) {
#pragma unroll
        for (int r = 0; r < 16; r++) dst[r] = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) dst = Elem<E>::mma(ko.c[j], qf.c[j], dst);
    };
    // mask of a partial score block
    auto mask_block = [&](f32x16& sc, int key0) {
        if constexpr (M::kRowIsRange) {
            fill_outside_range(sc, vis.lo, vis.hi, key0 + 4 * h, -INFINITY);
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                int key = key0 + 8 * (r / 4) + 4 * h + (r % 4);
                bool ok = (key < seq_len) && M::pred(q_pos, key, seq_len, p.margs);
                sc[r] = ok ? sc[r] : -INFINITY;
            }
        }
    };
    // mask and block max (scaled) of a score block
    auto prepare = [&](f32x16& sc, bool full, int key0) -> float {
        if (!full) mask_block(sc, key0);
        if constexpr (kGuard) return 0.f;
        float mx = sc[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
        return max_across_halves(mx) * scale;
    };
    // A operands of O^T += V^T P^T for step kb of the tile at `stage`: V^T blocks, read up front so
    // that their LDS latency hides behind the score MFMAs and the softmax of the step.
    // 16-bit: vt[s2][db] = transposed operand of keys 16*s2 .. 16*s2+15; fp32: read at use.
    struct VOperands {
        i16x4 lo[Elem<E>::k16 ? 2 : 1][Elem<E>::k16 ? DB : 1];
        i16x4 hi[Elem<E>::k16 ? 2 : 1][Elem<E>::k16 ? DB : 1];
    };
    auto load_v_operands = [&](VOperands& vo, const lds_char* stage, int kb) {
        if constexpr (Elem<E>::k16) {
            const lds_char* base = stage + v_lane + kb * 32 * VT::PITCH;
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    const lds_char* a0 = base + (16 * s2) * VT::PITCH + db * 64;
                    vo.lo[s2][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)a0);
                    vo.hi[s2][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(a0 + 8 * VT::PITCH));
                }
        }
    };
    // O^T += V^T P^T
    auto accumulate = [&](const f32x16& pr, const i32x4 (&packed)[2], const VOperands& vo, const lds_char* stage, int kb) {
        if constexpr (Elem<E>::k16) {
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                i32x4 bop;
                if constexpr (kGuard) {
                    bop = packed[s2];
                } else {
                    f32x8 ps;
#pragma unroll
                    for (int e = 0; e < 8; e++) ps[e] = pr[8 * s2 + e];
                    bop = Elem<E>::pack8(ps);
                }
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    i16x8 av = __builtin_shufflevector(vo.lo[s2][db], vo.hi[s2][db], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = Elem<E>::mma(__builtin_bit_cast(i32x4, av), bop, o[db]);
                }
            }
        } else {
            const lds_char* base = stage + v_lane + kb * 32 * VT::PITCH;
#pragma unroll
            for (int r = 0; r < 16; r++)
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    float a = *reinterpret_cast<const lds_float*>(base + (8 * (r / 4) + (r % 4)) * VT::PITCH + db * 128);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, pr[r], o[db], 0, 0, 0);
                }
        }
    };

    f32x16 s[2];         // scores of the current and of the next step
    KOperands ka;        // K operands of the next score block
    float mx_cur = 0.f;  // block max of s[current], already scaled
    const lds_char* lds0 = (const lds_char*)smem;
    // Q must have arrived before the loop: inside it the only vector-memory traffic is the async
    // tile loads, and the compiler must not place a wait for them in front of the first MFMA
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (p.scale_log2 < 0.f) {
#pragma unroll
            for (int e = 0; e < 4; e++) qf.c[j][e] ^= Elem<E>::k16 ? (int)0x80008000 : (int)0x80000000;
        }
        asm volatile("" ::"v"(qf.c[j]));
    }

    // One step: softmax of the current 32-key block and its share of O, with the scores of the next
    // block issued first.  With a tile resident ahead (LA >= 1) the step reads the next block
    // unconditionally — a wave's last step reads a stage whose contents it never uses — so that
    // between the rare rescale branch and the mask branch the step is one basic block, in which the
    // compiler places the softmax of this step among the score MFMAs of the next.
    auto step = [&](const lds_char* stage, const lds_char* stage_next, int kb, bool full, bool full_next, int k0) {
        f32x16& cur = s[kb & 1];
        f32x16& nxt = s[(kb + 1) & 1];
        if constexpr (!kGuard) {
            // rare path: raise the reference max and rescale what has been accumulated
            const bool raise = mx_cur > m_run + kRescaleTau;
            if (__builtin_amdgcn_ballot_w64(raise) != 0) {
                const float m_new = raise ? mx_cur : m_run;
                const float m_use_new = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = fast_exp2(m_use - m_use_new);
                m_run = m_new;
                m_use = m_use_new;
                l_run *= alpha;
    #pragma unroll
                for (int db = 0; db < DB; db++)
    #pragma unroll
                    for (int r = 0; r < 16; r++) o[db][r] *= alpha;
            }
        }
        const bool in_tile = kb + 1 < KB;
        const bool have_next = in_tile || LA >= 1;
        if (KB == 1 && LA >= 1) load_k_operands(ka, stage_next, 0);
        // V operands of this step: issued now, consumed after the softmax
        VOperands vo;
        load_v_operands(vo, stage, kb);
        __builtin_amdgcn_sched_barrier(0);
        // scores of the next step (operands already in registers) fly while this step's softmax runs
        if (have_next) scores(nxt, ka);
        float psum = 0.f;
        i32x4 pb[2];
        if constexpr (kGuard) {
            // P against the reference the row has, packed at once; the raw scores stay in `cur`
            auto softmax_block = [&]() {
                psum = 0.f;
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    f32x8 ps;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        ps[e] = fast_exp2(__builtin_fmaf(cur[8 * s2 + e], scale, -m_use));
                        psum += ps[e];
                    }
                    pb[s2] = Elem<E>::pack8(ps);
                }
            };
            softmax_block();
            // No block max on this path.  A row takes the max of its first block with a visible key as
            // reference and keeps it while the block sums stay below guard_above (far from the range of
            // P's type); a row without reference has guard_above = -1 and always comes here.
            const unsigned long long fired = __builtin_amdgcn_ballot_w64(psum > guard_above);
            if (fired != 0) {
                // the two lanes of a row (l and l ^ 32) hold half of its keys each and share its reference
                const bool fire = (((fired | (fired >> 32) | (fired << 32)) >> lane) & 1) != 0;
                float mx = cur[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, cur[r]);
                mx = max_across_halves(mx) * scale;
                const float m_new = fire ? fmaxf(m_run, mx) : m_run;
                const float m_use_new = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = fast_exp2(m_use - m_use_new);
                m_run = m_new;
                m_use = m_use_new;
                guard_above = (m_new == -INFINITY) ? -1.f : kGuardLimit;
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int r = 0; r < 16; r++) o[db][r] *= alpha;
                softmax_block();
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float pv = fast_exp2(__builtin_fmaf(cur[r], scale, -m_use));
                cur[r] = pv;
                psum += pv;
            }
        }
        l_run += psum;
        __builtin_amdgcn_sched_barrier(0);
        // K operands of the step after next, behind the score MFMAs that read the old ones
        if (kb + 2 < KB) {
            load_k_operands(ka, stage, kb + 2);
        } else if (KB > 1 && LA >= 1) {
            load_k_operands(ka, stage_next, kb + 2 - KB);
        }
        accumulate(cur, pb, vo, stage, kb);
        if constexpr (kGuard) {
            if (have_next) {
                if (in_tile) {
                    if (!full) mask_block(nxt, k0 + 32 * (kb + 1));
                } else {
                    if (!full_next) mask_block(nxt, k0 + TK);
                }
            }
        } else {
            if (have_next) mx_cur = in_tile ? prepare(nxt, full, k0 + 32 * (kb + 1)) : prepare(nxt, full_next, k0 + TK);
        }
    };

    int st_cur = NS - 1;  // LDS stage of tile i (advanced at the top of the loop)
    int st_issue = LA;    // LDS stage the next issued tile goes to
    for (int i = 0; i < n_tiles; i++) {
        // tiles <= i + LA have landed for every wave, and everyone is done with tile i - 1
        wait_async_tiles();
        __syncthreads();
        st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        if (i + LA + 1 < n_tiles) issue_tile(i + LA + 1, st_issue);
        if (i < ta || i >= tb) continue;
        const lds_char* stage = lds0 + st_cur * Lds::STAGE_BYTES;
        const lds_char* stage_next = lds0 + (st_cur + 1 == NS ? 0 : st_cur + 1) * Lds::STAGE_BYTES;
        const bool full = (i >= fa) && (i < fb);
        const bool full_next = (i + 1 >= fa) && (i + 1 < fb);
        const int k0 = (wg.start + i) * TK;
        if (LA == 0 || i == ta) {
            load_k_operands(ka, stage, 0);
            scores(s[0], ka);
            mx_cur = prepare(s[0], full, k0);
            // operands of the step after (with one step per tile they are read at the top of the step)
            if (KB > 1) load_k_operands(ka, stage, 1);
        }
#pragma unroll
        for (int kb = 0; kb < KB; kb++) step(stage, stage_next, kb, full, full_next, k0);
        if (KB & 1) s[0] = s[1];  // odd step count: the prefetched scores sit in the other buffer
    }

    // epilogue: O = acc / l, LSE2 = m + log2(l) (chill_fwd.py:288-289, 327-328)
    float l_tot = sum_across_halves(l_run);
    const float l_safe = (l_tot == 0.f) ? 1.f : l_tot;
    const float inv = 1.f / l_safe;
    const bool valid = q_pos < seq_len;
    const bool in_t = q_pos < p.T;
    if (in_t) {
        ET* orow = obase + (int64_t)q_pos * p.so.t;
        store_row_transposed<E, D>(orow, o, inv, valid, h);
        if (lse_base != nullptr && h == 0) lse_base[q_pos] = valid ? m_run + __log2f(l_safe) : 0.f;
    }
}

}  // namespace chill
#include "chill_fwd_regs.h"
#include "chill_fwd_fast.h"
#include "chill_fwd_small.h"
namespace chill {

// Shapes served by fwd_q_tile_fast (16-bit inputs, head dim 64 or 128, 64-key tiles with one resident
// ahead); fwd_q_tile stays behind it for the q-tiles whose sums leave the range it is exact in.
template <typename E, int D, int TK, int NS>
constexpr bool fwd_is_fast() {
    return CHILL_FWD_FAST && Elem<E>::k16 && (D == 64 || D == 128) && TK == 64 && NS >= 3;
}
template <typename E, int D, int TK, int NS>
constexpr int fwd_lds_bytes() {
    return NS * FwdLds<E, D, TK>::STAGE_BYTES + (fwd_is_fast<E, D, TK, NS>() ? kFwdFastFlagBytes : 0);
}

// Workgroups of four waves whose LDS ring leaves room for a second workgroup on the CU are compiled
// for 256 registers per wave, so that two of them share a CU: one computes while the other loads its
// first tiles or stores its result.
template <typename E, int D, int NW, int TK, int NS>
constexpr int fwd_waves_per_simd() {
    return (NW == 4 && Elem<E>::k16 && 2 * fwd_lds_bytes<E, D, TK, NS>() <= 160 * 1024) ? 2 : 1;
}

// One workgroup per (batch, head, PAIR of q-tiles): tile j from the end, then tile j from the
// start.  For causal-like masks the work of a q-tile grows with its index, so the two halves of a
// pair add up to the same amount for every workgroup and the grid finishes without a tail.
template <typename E, int D, int MASK, int NW, int TK, int NS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(fwd_waves_per_simd<E, D, NW, TK, NS>())))
void fwd_kernel(FwdParams p, int n_q_tiles, int total_items,
                                                      int wave_has_full_blocks, int paired) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // (unpaired q-tiles differ in length: the order for a grid that is resident at once)
    const int item = xcd_contiguous_item(blockIdx.x, total_items, paired ? 1 : fwd_waves_per_simd<E, D, NW, TK, NS>());
    if (item < 0) return;
    // paired: a workgroup takes q-tile j from the end and q-tile j from the start (equal work under
    // causal-like masks); unpaired: one q-tile per workgroup, last tiles first
    const int per_head = paired ? (n_q_tiles + 1) / 2 : n_q_tiles;
    const int bh = item / per_head;
    const int j = item % per_head;
    const int b = bh / p.H;
    const int hd = bh % p.H;
    const int qt_hi = n_q_tiles - 1 - j;
    if constexpr (fwd_is_fast<E, D, TK, NS>()) {
        fwd_fast_q_tiles<E, D, MASK, NW, TK, NS>(p, smem, b, hd, qt_hi, (paired && j != qt_hi) ? j : -1,
                                                 wave_has_full_blocks);
    } else {
        fwd_q_tile<E, D, MASK, NW, TK, NS>(p, smem, b, hd, qt_hi, wave_has_full_blocks);
        if (paired && j != qt_hi) {
            __syncthreads();  // the LDS ring is reused
            fwd_q_tile<E, D, MASK, NW, TK, NS>(p, smem, b, hd, j, wave_has_full_blocks);
        }
    }
}

// Launcher for one (element type, head dim); dispatches on the mask id and takes the tile shape
// from the static table.
// fewer paired workgroups than an MI355X has CUs: launch one q-tile per workgroup (measured on causal
// shapes: 16-35 % faster below the threshold, 7-16 % slower at two to four times it)
constexpr int kPairedMinWorkgroups = 256;

// One (mask, tile shape): SHORT selects the table row for short sequences.
template <typename E, int D, int MASK_ID, bool SHORT>
int launch_fwd_shape(const FwdParams& p, hipStream_t stream) {
    constexpr int kRowFor = SHORT ? 1 : kLongSequence;
    constexpr TileConfig cfg = fwd_tile_config(MASK_ID, D, Elem<E>::kDType, kRowFor);
    static_assert(cfg.rows == cfg.waves * 32, "one wave owns 32 rows");
    constexpr int NS = fwd_stages(MASK_ID, D, Elem<E>::kDType, kRowFor);
    static_assert(cfg.lds_bytes == NS * FwdLds<E, D, cfg.streamed>::STAGE_BYTES, "table and kernel disagree on LDS");
    constexpr int kLdsBytes = fwd_uses_regs(D, Elem<E>::kDType) ? cfg.lds_bytes : fwd_lds_bytes<E, D, cfg.streamed, NS>();
    const int n_q_tiles = cdiv(p.T, cfg.rows);
    // pairing q-tiles balances long causal runs; with few workgroups it only halves the number of
    // CUs that get work
    const bool paired = (int64_t)p.B * p.H * ((n_q_tiles + 1) / 2) >= kPairedMinWorkgroups;
    const int64_t total64 = (int64_t)p.B * p.H * (paired ? (n_q_tiles + 1) / 2 : n_q_tiles);
    if (total64 > ((int64_t)1 << 30)) return CHILL_ERR_TOO_LARGE;
    const int total = (int)total64;
    dim3 grid(cdiv(total, 8) * 8), block(cfg.waves * 64);
    void (*kern)(FwdParams, int, int, int, int);
    if constexpr (fwd_uses_regs(D, Elem<E>::kDType))
        kern = fwd_regs_kernel<E, D, MASK_ID, cfg.streamed, NS>;
    else
        kern = fwd_kernel<E, D, MASK_ID, cfg.waves, cfg.streamed, NS>;
    const bool hfb = Mask<MASK_ID>::has_full_blocks(32, cfg.streamed, p.T, p.margs);
    if (kLdsBytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kLdsBytes) != hipSuccess)
            return CHILL_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, grid, block, kLdsBytes, stream, p, n_q_tiles, total, hfb ? 1 : 0, paired ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

// A launch far too small for the chip: 32 query rows per workgroup, the keys split over its waves.
template <typename E, int D, int MASK_ID>
int launch_fwd_small(const FwdParams& p, hipStream_t stream) {
    constexpr int kLdsOne = fwd_small_lds_bytes(D, Elem<E>::kDType);
    const int n_q_tiles = cdiv(p.T, 32);
    // (at most kComputeUnits / 4 * 4 * 32 q-tiles by fwd_takes_small)
    bool two = false;
    if constexpr (small_fits_two_tiles(kLdsOne)) two = small_takes_two_tiles((long long)p.B * p.H * n_q_tiles);
    const int total = p.B * p.H * (two ? (n_q_tiles + 1) / 2 : n_q_tiles);
    const int lds_bytes = two ? 2 * kLdsOne : kLdsOne;
    void (*kern)(FwdParams, int, int, int) = fwd_small_kernel<E, D, MASK_ID, 1>;
    if constexpr (small_fits_two_tiles(kLdsOne)) {
        if (two) kern = fwd_small_kernel<E, D, MASK_ID, 2>;
    }
    const bool hfb = Mask<MASK_ID>::has_full_blocks(32, 32, p.T, p.margs);
    if (lds_bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds_bytes) != hipSuccess)
            return CHILL_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, dim3(total), dim3(kFwdSmallWaves * 64 * (two ? 2 : 1)), lds_bytes, stream, p, n_q_tiles, total,
                       hfb ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

template <typename E, int D>
int launch_fwd(const FwdParams& p, int mask_id, hipStream_t stream) {
    // the async loader keeps per-lane global offsets in 32 bits
    const int64_t max_stride = p.sk.t > p.sv.t ? p.sk.t : p.sv.t;
    if (max_stride * Elem<E>::kBytes * 256 >= ((int64_t)1 << 31)) return CHILL_ERR_TOO_LARGE;
    int status = CHILL_ERR_BAD_MASK;
    CHILL_DISPATCH_MASK(mask_id, {
        // the table has a row of its own for short sequences and small grids where that row differs
        constexpr bool has_short_row = fwd_tile_config(MASK_ID, D, Elem<E>::kDType, 1).waves !=
                                       fwd_tile_config(MASK_ID, D, Elem<E>::kDType).waves;
        bool small = false;
        if constexpr (D * Elem<E>::kBytes <= 512) small = fwd_takes_small(MASK_ID, (long long)p.B * p.H, p.T, D, Elem<E>::kDType);
        if (small) {
            if constexpr (D * Elem<E>::kBytes <= 512) status = launch_fwd_small<E, D, MASK_ID>(p, stream);
        } else if constexpr (has_short_row) {
            const bool short_row = fwd_takes_short_row(MASK_ID, mask_band_keys(MASK_ID, p.margs.a0, p.margs.a1),
                                                       (long long)p.B * p.H, p.T);
            status = short_row ? launch_fwd_shape<E, D, MASK_ID, true>(p, stream) : launch_fwd_shape<E, D, MASK_ID, false>(p, stream);
        } else {
            status = launch_fwd_shape<E, D, MASK_ID, false>(p, stream);
        }
    });
    return status;
}

}  // namespace chill
