// Forward q-tile for 16-bit inputs, head dims 64 and 128: the same algorithm, data layout and tile
// skipping as fwd_q_tile (chill_fwd_kernel.h; reference chill_attention/chill_fwd.py:21-359), with
// the online softmax reduced to what a matrix-bound loop can carry:
//
//   * Q is multiplied by scale * log2(e) once, when it is loaded (the reference's prescale_qk,
//     chill_fwd.py:120-127), so an accumulator of S^T = K Q^T already holds the exponent;
//   * a row takes ONE reference m0, the max over its first visible block(s), before the loop; the
//     score MFMA chains start from an accumulator block filled with -m0, so the exponent minus the
//     reference comes out of the matrix pipe and P = exp2(acc) costs one instruction per entry;
//   * the reference is raised only where a row asks for it.  O and LSE2 do not depend on it beyond
//     rounding as long as the sums stay inside the range of the types, so nothing is compared or rescaled
//     block by block: a wave tests one sum per block (fp16: the lane's sum of P over the block against
//     2^15) or per tile (bf16: the row sum against 2^40), and if any of its rows is above, a rare
//     out-of-line block raises the references to the largest exponent at hand and rescales O^T, the row
//     sums and the scores in flight (gen_raise in gen_fwd_loop.py; the same in plain_step below).
//     Scores that climb by more than ~15 (fp16) / ~40 (bf16) log2 units above a row's reference are what
//     it takes.  A row whose sum still ends outside [kLo, kHi] (a jump of more than ~80 units inside one
//     tile, a NaN) marks the q-tile, and the kernel runs such a q-tile again through fwd_q_tile, whose
//     softmax follows the running max block by block;
//   * a step (32 keys) is software-pipelined two deep: while the matrix pipe runs O^T += V^T P(g)^T
//     and then S(g+2)^T, the vector ALU turns S(g+1) into P(g+1) and the LDS reads of the operands
//     of the other phase are in flight, every MFMA followed by its share of each.
//
// A wave works on its own range of 32-key BLOCKS (tile_range with 32-key tiles), inside the
// workgroup's ring of 64-key tiles.
#pragma once

#include "chill_fwd_kernel.h"
#include "chill_fwd_loop.inc"

namespace chill {

typedef int i32x16 __attribute__((ext_vector_type(16)));

// shapes whose steady state runs in the generated loop (gen_fwd_loop.py)
template <typename E, int D, int NW, int NS>
constexpr bool fwd_has_generated_loop() {
    return Elem<E>::k16 && ((D == 128 && NW == 8 && NS == 4) || (D == 64 && NW == 4 && NS == 3));
}

template <typename E>
struct FastSoftmaxLimits;
template <>
struct FastSoftmaxLimits<bf16_t> {
    static constexpr float kLo = 0x1p-60f, kHi = 0x1p60f;
    static constexpr float kBlockHi = 0.f;
    static constexpr float kRaiseAbove = 0x1p40f;   // a lane's sum over a block that has the reference raised
};
template <>
struct FastSoftmaxLimits<f16_t> {
    static constexpr float kLo = 0x1p-6f, kHi = 0x1p60f;
    static constexpr float kBlockHi = 32768.f;      // every P of a block stays below 65504 while the lane's sum does
    static constexpr float kRaiseAbove = kBlockHi;
};

// bytes behind the ring: one flag per wave for the workgroup's vote on running the q-tile again
constexpr int kFwdFastFlagBytes = 64;

// x * f for the 8 elements of a 16-byte chunk
template <typename E>
__device__ __forceinline__ i32x4 scale_chunk(i32x4 c, float f) {
    typedef typename Elem<E>::type ET;
    typedef ET etx8 __attribute__((ext_vector_type(8)));
    f32x8 x = __builtin_convertvector(__builtin_bit_cast(etx8, c), f32x8);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] *= f;
    return Elem<E>::pack8(x);
}


// true if `mine` is true for any wave of the workgroup; flags = one int per wave in LDS
template <int NW>
__device__ __forceinline__ bool workgroup_any(bool mine, char* flags) {
    volatile int* f = reinterpret_cast<volatile int*>(flags);
    if ((threadIdx.x & 63) == 0) f[threadIdx.x >> 6] = mine ? 1 : 0;
    __syncthreads();
    int any = 0;
#pragma unroll
    for (int w = 0; w < NW; w++) any |= f[w];
    __syncthreads();  // the flags are reused
    return __builtin_amdgcn_readfirstlane(any) != 0;  // (the same in every lane: say so to the compiler)
}

// The q-tiles qt_a and then qt_b (-1: none) of one head, start to finish.  While the rows of one q-tile
// are normalised and stored, the first K/V tiles and the Q rows of the next one are already on their
// way.  A q-tile in which a row left the range the reference-free softmax is exact in is computed
// again by fwd_q_tile.
template <typename E, int D, int MASK, int NW, int TK, int NS>
__device__ __forceinline__ void fwd_fast_q_tiles(const FwdParams& p, char* smem, int b, int hd, int qt_a, int qt_b,
                                                 int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    using M = Mask<MASK>;
    typedef FwdLds<E, D, TK> Lds;
    typedef typename Lds::KT KT;
    typedef typename Lds::VT VT;
    typedef FastSoftmaxLimits<E> Lim;
    static_assert(Elem<E>::k16 && (D == 64 || D == 128), "16-bit inputs, head dim 64 or 128");
    static_assert(TK == 64 && NS >= 3, "64-key tiles; one resident ahead of the one being consumed");
    constexpr int TQ = NW * 32;
    constexpr int NT = NW * 64;
    constexpr int KB = TK / 32;       // steps per tile
    constexpr int DB = D / 32;
    constexpr int NJ = KT::CH / 2;
    constexpr int FL = NS - 3;        // tiles in flight beyond the one the barrier certifies
    const int hkv = hd / p.group;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    ET* obase = reinterpret_cast<ET*>(p.o) + b * p.so.b + hd * p.so.h;
    float* lse_base = p.lse ? p.lse + b * p.lse_b + hd * p.lse_h : nullptr;
    const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h;
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;

    AsyncPaddedLoader<E, D, rowwise_pad<E, D>(), TK, NT> load_k;
    AsyncPaddedLoader<E, D, transposed_pad<E, D>(), TK, NT> load_v;
    load_k.init(p.sk.t, wave, lane);
    load_v.init(p.sv.t, wave, lane);
    // every wave issues at least this many loads per tile
    constexpr int kLoadsPerTile = decltype(load_k)::SLABS / NW + decltype(load_v)::SLABS / NW;
    // tile `tile` (absolute index along the keys) into LDS stage st_index
    auto issue_tile = [&](int tile, int st_index) {
        int k0 = tile * TK;
        char* st = smem + st_index * Lds::STAGE_BYTES;
        load_k.issue(kptr + (int64_t)k0 * p.sk.t, p.sk.t, p.T - k0, st, wave, lane);
        load_v.issue(vptr + (int64_t)k0 * p.sv.t, p.sv.t, p.T - k0, st + Lds::K_BYTES, wave, lane);
    };

    // per-lane LDS offsets inside a stage; everything else is an immediate
    const int k_lane = n * KT::PITCH + h * 16;
    const int r16 = lane & 15, colgrp = (lane >> 4) & 1;
    const int v_lane = Lds::K_BYTES + (4 * h + (r16 >> 2)) * VT::PITCH + (16 * colgrp + 4 * (r16 & 3)) * 2;
    const lds_char* lds0 = (const lds_char*)smem;

    struct KOperands {
        i32x4 c[NJ];
    };
    struct VOperands {
        i16x4 lo[2][DB];
        i16x4 hi[2][DB];
    };
    auto k_read = [&](KOperands& ko, const lds_char* stage, int kb) {
        const lds_char* base = stage + k_lane + kb * 32 * KT::PITCH;
#pragma unroll
        for (int j = 0; j < NJ; j++) ko.c[j] = *reinterpret_cast<const lds_i32x4*>(base + j * 32);
    };
    auto v_read = [&](VOperands& vo, const lds_char* stage, int kb) {
        const lds_char* base = stage + v_lane + kb * 32 * VT::PITCH;
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
            for (int db = 0; db < DB; db++) {
                const lds_char* a0 = base + (16 * s2) * VT::PITCH + db * 64;
                vo.lo[s2][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)a0);
                vo.hi[s2][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(a0 + 8 * VT::PITCH));
            }
    };

    // What is on its way for the next q-tile: the tiles of its hull wg_pre (the first NS - 1 of them,
    // tile i in stage i) and its Q rows in qf.
    Resident<E, D> qf;
    TileRange wg_pre = {0, 0, 0, 0};
    auto prefetch = [&](int qt) {
        const int qb = qt * TQ;
        wg_pre = TileRange{0, 0, 0, 0};
        if (qb >= seq_len) return;
        wg_pre = tile_range<MASK, true>(qb, TQ, TK, seq_len, false, p.margs);
#pragma unroll
        for (int i = 0; i <= 1 + FL; i++)
            if (wg_pre.start + i < wg_pre.end) issue_tile(wg_pre.start + i, i);
        const int qw = qb + 32 * wave;
        load_resident<E, D>(qf, qptr + (int64_t)qw * p.sq.t, p.sq.t, p.T - qw, lane);
    };
    prefetch(qt_a);

#pragma nounroll
    for (int item = 0; item < 2; item++) {
        const int qt = item == 0 ? qt_a : qt_b;
        const int qt_next = item == 0 ? qt_b : -1;
        if (qt < 0) break;
        const int qb = qt * TQ;
        if (qb >= seq_len) {
            // nothing attends here: the output rows are defined to be zero (chill.py:96, chill_fwd.py:70-71)
            int nrows = imin(TQ, p.T - qb);
            zero_rows<E, D, NT>(obase, p.so.t, qb, nrows, tid);
            if (lse_base)
                for (int i = tid; i < nrows; i += NT) lse_base[qb + i] = 0.f;
            if (qt_next >= 0) prefetch(qt_next);
            continue;
        }
        const TileRange wg = {uniform(wg_pre.start), uniform(wg_pre.end), 0, 0};
        const int n_tiles = wg.end - wg.start;
        const int qw = qb + 32 * wave;

        // this wave's 32-key blocks, as steps counted from the first block of the workgroup's first tile
        int g0 = 0, g1 = 0, f0 = 0, f1 = 0;
        if (qw < seq_len) {
            const TileRange wr =
                tile_range<MASK, true>(qw, 32, 32, seq_len, M::has_full_blocks(32, 32, p.T, p.margs), p.margs);
            const int base = wg.start * KB;
            g0 = imax(wr.start - base, 0);
            g1 = imin(wr.end - base, n_tiles * KB);
            f0 = wr.full_start - base;
            f1 = wr.full_end - base;
        }

        f32x16 o[DB];
#pragma unroll
        for (int i = 0; i < DB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[i][r] = 0.f;
        float l_run = 0.f;   // this lane's share of the row sum
        float m0 = 0.f;      // the row's reference (log2 domain, scale included)
        const int q_pos = qw + n;
        const Range vis = visible_range<MASK, true>(q_pos, seq_len, p.margs);  // the keys this lane's row sees

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

        // Q: wait for it, fold the scale in (a negative scale needs nothing special here)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            qf.c[j] = scale_chunk<E>(qf.c[j], p.scale_log2);
            asm volatile("" : "+v"(qf.c[j]));
        }

        f32x16 mneg;  // the accumulator block the score chains start from: -m0 everywhere
#pragma unroll
        for (int r = 0; r < 16; r++) mneg[r] = 0.f;

        bool have_ref = false;  // wave-uniform: the rows have their reference
        // One step outside the generated loop, from the scores to O: block g of the wave (the first one
        // also settles the row's reference).  Not pipelined: the first and the last few blocks of a wave,
        // and every block that needs the mask, come here.
        auto plain_step = [&](const lds_char* stage, int kb, int g) {
            KOperands ka;
            k_read(ka, stage, kb);
            f32x16 sc = Elem<E>::mma(ka.c[0], qf.c[0], mneg);
#pragma unroll
            for (int j = 1; j < NJ; j++) sc = Elem<E>::mma(ka.c[j], qf.c[j], sc);
            if (g < f0 || g >= f1) mask_block(sc, (wg.start * KB + g) * 32);
            if (!have_ref) {
                have_ref = true;
                float mx = sc[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
                mx = max_across_halves(mx);
                m0 = (mx == -INFINITY) ? 0.f : mx;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    mneg[r] = -m0;
                    sc[r] -= m0;
                }
                asm volatile("" : "+v"(mneg));  // sixteen registers, not one value the compiler may splat again
            }
            VOperands vo;
            v_read(vo, stage, kb);
            float psum = 0.f;
            i32x4 pb[2];
            auto softmax_block = [&]() {
                psum = 0.f;
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    f32x8 ps;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        ps[e] = fast_exp2(sc[8 * s2 + e]);
                        psum += ps[e];
                    }
                    pb[s2] = Elem<E>::pack8(ps);
                }
            };
            softmax_block();
            // a block whose sum leaves the range of P's type (fp16), or that takes the row sum far up (bf16): the
            // reference of the rows is raised to the largest exponent of the block, as the generated loop does
            if (__builtin_amdgcn_ballot_w64(psum > Lim::kRaiseAbove) != 0) {
                float mx = sc[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
                const float d = fmaxf(max_across_halves(mx), 0.f);
                const float alpha = fast_exp2(-d);
                m0 += d;
                l_run *= alpha;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    mneg[r] = -m0;
                    sc[r] -= d;
                }
                asm volatile("" : "+v"(mneg));
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int r = 0; r < 16; r++) o[db][r] *= alpha;
                softmax_block();
            }
            l_run += psum;
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    i16x8 av = __builtin_shufflevector(vo.lo[s2][db], vo.hi[s2][db], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = Elem<E>::mma(__builtin_bit_cast(i32x4, av), pb[s2], o[db]);
                }
        };

        // Tiles [i_lo, i_hi) go to the generated loop: both blocks inside the wave's range and
        // predicate-free.
        int i_lo = (imax(g0, f0) + KB - 1) / KB;
        int i_hi = imin(imin(g1, f1) / KB, n_tiles);
        // a tile that ends past T is zero-filled by its loader, which the generated loop does not do
        if (p.T % TK != 0) i_hi = imin(i_hi, p.T / TK - wg.start - (NS - 1));
        if (!fwd_has_generated_loop<E, D, NW, NS>() || g1 <= g0 || i_hi < i_lo) i_lo = i_hi = 0;

        int st_cur = NS - 1;  // LDS stage of tile i (advanced at the top of the loop)
        // Tiles <= i + 1 have landed for every wave, and everyone is done with tile i - 1.  The first wait
        // of a q-tile is for everything: the stores of the q-tile before are among what is outstanding,
        // and they do not complete in order with the loads.
        auto ring_top = [&](int i, bool issue) {
            if (FL > 0 && i > 0 && i + 1 + FL < n_tiles)
                wait_async_tiles_except<FL * kLoadsPerTile>();
            else
                wait_async_tiles();
            __syncthreads();
            st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
            if (issue && i + NS - 1 < n_tiles) issue_tile(wg.start + i + NS - 1, st_cur == 0 ? NS - 1 : st_cur - 1);
        };
        auto plain_tile = [&](int i) {
            ring_top(i, true);
            const lds_char* stage = lds0 + st_cur * Lds::STAGE_BYTES;
#pragma unroll
            for (int kb = 0; kb < KB; kb++) {
                const int g = i * KB + kb;
                if (g >= g0 && g < g1) plain_step(stage, kb, g);
            }
        };
        int i = 0;
        for (; i < i_lo || (i_lo == i_hi && i < n_tiles); i++) plain_tile(i);
        if constexpr (fwd_has_generated_loop<E, D, NW, NS>()) {
            if (i_hi > i_lo) {
                ring_top(i_lo, false);  // the generated loop issues the tile that is due here
                if (!have_ref) {
                    // the wave starts here: the reference comes from its first block, whose scores the
                    // loop computes again
                    have_ref = true;
                    KOperands ka;
                    k_read(ka, lds0 + st_cur * Lds::STAGE_BYTES, 0);
                    f32x16 sc = Elem<E>::mma(ka.c[0], qf.c[0], mneg);
#pragma unroll
                    for (int j = 1; j < NJ; j++) sc = Elem<E>::mma(ka.c[j], qf.c[j], sc);
                    float mx = sc[0];
#pragma unroll
                    for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
                    m0 = max_across_halves(mx);
#pragma unroll
                    for (int r = 0; r < 16; r++) mneg[r] = -m0;
                    asm volatile("" : "+v"(mneg));
                }
                // (all of these are the same in every lane; uniform() says so where the compiler has lost track)
                int cnt = uniform(i_hi - i_lo);
                int rem = uniform(n_tiles - i_lo - 2);   // tiles behind the one the last barrier certified
                const unsigned lds_base = lds_address(smem);
                unsigned cur = uniform(lds_base + st_cur * Lds::STAGE_BYTES);   // stage of tile i_lo
                const int t_issue = uniform((wg.start + i_lo + NS - 1) * TK);  // first key of the next tile to load
                const ET* kb = kptr + (int64_t)t_issue * p.sk.t;
                const ET* vb = vptr + (int64_t)t_issue * p.sv.t;
                const unsigned kstep = (unsigned)(TK * p.sk.t * Elem<E>::kBytes), vstep = (unsigned)(TK * p.sv.t * Elem<E>::kBytes);
                const unsigned w1024 = wave * 1024;
                // Q as the loop takes it: sixteen registers per operand
                i32x16 q0, q1;
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        q0[4 * j + e] = qf.c[j][e];
                        q1[4 * j + e] = qf.c[(NJ > 4 ? 4 : 0) + j][e];
                    }
                const float block_hi = Lim::kBlockHi;
                constexpr bool kBf16 = std::is_same<E, bf16_t>::value;
                static_assert(decltype(load_k)::PER_WAVE == 3 && decltype(load_v)::PER_WAVE == 3, "three loads per wave and tile");
                if constexpr (D == 128 && kBf16) {
                    CHILL_FWD_LOOP_BF16_128_8_4(o[0], o[1], o[2], o[3], l_run, cnt, rem, cur, kb, vb, mneg, q0, q1, k_lane,
                                                v_lane, load_k.goff[0], load_k.goff[1], load_k.goff[2], load_v.goff[0],
                                                load_v.goff[1], load_v.goff[2], lds_base, kstep, vstep, w1024, wave);
                } else if constexpr (D == 128) {
                    CHILL_FWD_LOOP_F16_128_8_4(o[0], o[1], o[2], o[3], l_run, cnt, rem, cur, kb, vb, mneg, q0, q1, k_lane,
                                               v_lane, load_k.goff[0], load_k.goff[1], load_k.goff[2], load_v.goff[0],
                                               load_v.goff[1], load_v.goff[2], lds_base, kstep, vstep, w1024, wave, block_hi);
                } else if constexpr (kBf16) {
                    CHILL_FWD_LOOP_BF16_64_4_3(o[0], o[1], l_run, cnt, rem, cur, kb, vb, mneg, q0, k_lane, v_lane,
                                               load_k.goff[0], load_k.goff[1], load_k.goff[2], load_v.goff[0], load_v.goff[1],
                                               load_v.goff[2], lds_base, kstep, vstep, w1024, wave);
                } else {
                    CHILL_FWD_LOOP_F16_64_4_3(o[0], o[1], l_run, cnt, rem, cur, kb, vb, mneg, q0, k_lane, v_lane,
                                              load_k.goff[0], load_k.goff[1], load_k.goff[2], load_v.goff[0], load_v.goff[1],
                                              load_v.goff[2], lds_base, kstep, vstep, w1024, wave, block_hi);
                }
                // the loop raises the reference where a row asks for it: what it leaves in the chain start is the
                // reference from here on
                m0 = -mneg[0];
                st_cur = (st_cur + (i_hi - i_lo - 1)) % NS;
                i = i_hi;
            }
        }
        for (; i < n_tiles; i++) plain_tile(i);

        // the ring is free once every wave is here: start on the next q-tile before this one is stored
        if (qt_next >= 0) {
            __syncthreads();
            prefetch(qt_next);
        }

        // epilogue: O = acc / l, LSE2 = m0 + log2(l) (chill_fwd.py:288-289, 327-328)
        const float l_tot = sum_across_halves(l_run);
        const float l_safe = (l_tot == 0.f) ? 1.f : l_tot;
        const float inv = 1.f / l_safe;
        const bool valid = q_pos < seq_len;
        const bool in_t = q_pos < p.T;
        if (in_t) {
            ET* orow = obase + (int64_t)q_pos * p.so.t;
            store_row_transposed<E, D>(orow, o, inv, valid, h);
            if (lse_base != nullptr && h == 0)
                lse_base[q_pos] = valid ? (l_tot == 0.f ? -INFINITY : m0 + __log2f(l_tot)) : 0.f;
        }
        // a row that sees keys must end with a sum inside the range (a NaN fails the comparison too)
        const bool bad = (vis.lo <= vis.hi) && !(l_tot >= Lim::kLo && l_tot <= Lim::kHi);
        const bool again = __builtin_amdgcn_ballot_w64(bad) != 0;
        if (workgroup_any<NW>(again, smem + NS * Lds::STAGE_BYTES)) {
            // rare: give the ring to the kernel whose softmax follows the running max, then start over on
            // the next q-tile
            wait_async_tiles();
            __syncthreads();
            fwd_q_tile<E, D, MASK, NW, TK, 3>(p, smem, b, hd, qt, wave_has_full_blocks);
            __syncthreads();
            if (qt_next >= 0) prefetch(qt_next);
        }
    }
}

}  // namespace chill
