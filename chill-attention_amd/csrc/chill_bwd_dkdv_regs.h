// dK/dV with the accumulators in hand-managed accumulation registers (16-bit inputs).
//
// A workgroup of 4 waves (one per SIMD, so each wave may use the whole 512-entry register file)
// owns 4 * CB * 32 key rows, CB blocks of 32 per wave.  A wave keeps its K rows in registers as MFMA
// B operands (the V rows stay in LDS: both would not fit beside the score blocks) and its dK^T / dV^T
// accumulators (CB x D/32 blocks of 16 registers each) in the accumulation registers under fixed
// names (see the hand-placed MFMA helpers in chill_device.h).  Streamed through the LDS ring: Q and
// dO tiles of 32 query rows with their LSE2 / delta, for every query head of the GQA group in turn
// (chill_bwd_dkdv.py:156).
//
//   S = Q K^T, dP = dO V^T, P = exp2(S * scale - LSE2), dS = P o (dP - delta),
//   dV^T += dO^T P, dK^T += Q^T dS, finally dK *= sm_scale            (chill_bwd_dkdv.py:362-403, 230)
//
// CB = 1, D = 256 (512-byte rows) is the shipped dK/dV kernel of that shape: 2 x 8 accumulator blocks
// are exactly the 256 accumulation registers, which the compiler cannot keep there by itself (its
// version of this kernel spills 2400 registers to scratch and runs 40x slower).
// CB = 2, D = 64 / 128 is the dK/dV kernel of long sequences at those head dims (chill_tiles.h:
// dkdv_takes_regs): every streamed operand fetched from LDS feeds two MFMAs and K is never re-read, at
// D = 128 76 LDS reads per 64 MFMAs where the paired kernel needs 146.  Its runs of predicate-free tiles
// go through a generated, hazard-checked loop (gen_bwd_loop.py -> chill_bwd_loop.inc); with the
// compiler's schedule the shape was no faster than the paired kernel (a lone wave hides its vector work
// only behind its own MFMAs).
//
// Every translation unit that instantiates this kernel is checked (tests/test_abi.py) for the
// compiler keeping out of the accumulation registers the kernel names itself.
#pragma once

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"
#include "chill_bwd_loop.inc"

namespace chill {

// Shapes whose runs of predicate-free tiles go through the generated loop (gen_bwd_loop.py).  Such a kernel
// keeps V NEGATED in LDS: the dP chain of a block starts from delta and ends as dP' = delta - dO V^T, so that
// dS' = P dP' = -dS costs one multiplication per entry, and dK^T is accumulated with the opposite sign and
// stored times -sm_scale.
template <typename E, int D, int CB, int NS>
constexpr bool dkdv_has_generated_loop() {
    return Elem<E>::k16 && (D == 128 || D == 64) && CB == 2 && NS == 4;
}

template <typename E, int D, int MASK, int CB, int NS>
__global__ __launch_bounds__(256) void dkdv_regs_kernel(BwdParams p, int n_k_tiles, int total_items,
                                                       int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    static_assert(Elem<E>::k16, "16-bit element types");
    typedef LdsTile<E, D> L;
    constexpr int NW = 4;
    constexpr int NT = NW * 64;
    constexpr int KPW = 32 * CB;     // key rows per wave: CB 32-key blocks
    constexpr int TKR = NW * KPW;    // key rows per workgroup
    constexpr int TQS = 32;          // streamed query rows per tile
    constexpr int DB = (D + 31) / 32;
    constexpr int NJ = Resident<E, D>::NJ;
    constexpr int TILE_BYTES = L::bytes(TQS);
    constexpr int VEC_BYTES = TQS * 4;
    constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * VEC_BYTES;  // Q, dO, LSE2, delta
    constexpr int V_BYTES = L::bytes(TKR);                       // the workgroup's V rows, then the ring
    constexpr int LA = NS - 2;  // tiles resident ahead of the one being consumed
    static_assert(NS >= 2 && NS <= 4, "ring stages");
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int item = xcd_contiguous_item(blockIdx.x, total_items);
    if (item < 0) return;
    const int bh = item / n_k_tiles;
    // key tiles first-to-last: for causal-like masks the longest run first
    const int ktile = item % n_k_tiles;
    const int b = bh / p.H_kv;
    const int hkv = bh % p.H_kv;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    const int kb0 = ktile * TKR;
    ET* dkbase = reinterpret_cast<ET*>(p.dk) + b * p.sdk.b + hkv * p.sdk.h;
    ET* dvbase = reinterpret_cast<ET*>(p.dv) + b * p.sdv.b + hkv * p.sdv.h;
    if (kb0 >= seq_len) {
        int nrows = imin(TKR, p.T - kb0);
        zero_rows<E, D, NT>(dkbase, p.sdk.t, kb0, nrows, tid);
        zero_rows<E, D, NT>(dvbase, p.sdv.t, kb0, nrows, tid);
        return;
    }

    const TileRange wg = tile_range<MASK, false>(kb0, TKR, TQS, seq_len, false, p.margs);
    const int n_tiles = wg.end - wg.start;
    const int n_iters = n_tiles * p.group;

    AsyncSwizzledLoader<E, D, TQS, NT> load_q, load_do;
    load_q.init(p.sq.t, wave, lane);
    load_do.init(p.sdo.t, wave, lane);
    // iteration it = (group head g, q-tile): stage it % NS
    auto issue_iter = [&](int it, int st_index) {
        const int g = it / n_tiles;
        const int q0 = (wg.start + it % n_tiles) * TQS;
        const int hq = hkv * p.group + g;
        char* st = smem + V_BYTES + st_index * STAGE_BYTES;
        const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hq * p.sq.h;
        const ET* doptr = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hq * p.sdo.h;
        load_q.issue(qptr + (int64_t)q0 * p.sq.t, p.T - q0, st, wave, lane);
        load_do.issue(doptr + (int64_t)q0 * p.sdo.t, p.T - q0, st + TILE_BYTES, wave, lane);
        if (wave == NW - 1 && lane < TQS) {
            // LSE2 and delta of the tile's rows; rows past the end of the tensor read as zero
            const float* lse = p.lse + b * p.lse_b + hq * p.lse_h + q0;
            const float* del = p.delta + b * p.delta_b + hq * p.delta_h + q0;
            char* vec = st + 2 * TILE_BYTES;
            if (q0 + lane < p.T) {
                async_load4(lse, lane * 4, lds_address(vec));
                async_load4(del, lane * 4, lds_address(vec + VEC_BYTES));
            } else {
                reinterpret_cast<float*>(vec)[lane] = 0.f;
                reinterpret_cast<float*>(vec + VEC_BYTES)[lane] = 0.f;
            }
        }
    };
    {
        AsyncSwizzledLoader<E, D, TKR, NT> load_v;
        const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;
        load_v.init(p.sv.t, wave, lane);
        load_v.issue(vptr + (int64_t)kb0 * p.sv.t, p.T - kb0, smem, wave, lane);
    }
#pragma unroll
    for (int i = 0; i <= LA; i++)
        if (i < n_iters) issue_iter(i, i);

    constexpr bool kGen = dkdv_has_generated_loop<E, D, CB, NS>();
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const int kw = kb0 + KPW * wave;
    OperandOffsets<E, D> ofs;
    ofs.init(lane);
    if constexpr (kGen) {
        // every lane flips the sign of the V chunks it has loaded itself, once they are there (the first barrier
        // of the loop stands between this and the first read of V)
        wait_async_tiles();
        constexpr int PER = TKR * L::CH / NT;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            i32x4* at = reinterpret_cast<i32x4*>(smem) + (i * NW + wave) * 64 + lane;
            i32x4 x = *at;
#pragma unroll
            for (int e = 0; e < 4; e++) x[e] ^= (int)0x80008000;
            *at = x;
        }
    }
    Resident<E, D> kf[CB];
#pragma unroll
    for (int c = 0; c < CB; c++)
        load_resident<E, D>(kf[c], kptr + (int64_t)(kw + 32 * c) * p.sk.t, p.sk.t, p.T - kw - 32 * c, lane);

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    // (key rows of the wave at and beyond seq_len are computed like the others and stored as zeros)
    if (kw < seq_len) wr = tile_range_rows_discarded<MASK, false>(kw, KPW, TQS, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    // accumulation registers: dV^T block (c, db) at a[16 * (c * DB + db)], dK^T blocks after them
    constexpr int DV_BASE = 0, DK_BASE = CB * DB * 16;
    static_assert(2 * CB * DB * 16 <= 256, "accumulators exceed the accumulation registers");
    agpr_reserve();
    int tok = agpr_zero<0, 2 * CB * DB * 16>();
    const float scale = p.scale_log2;
    const float masked_score = scale < 0.f ? INFINITY : -INFINITY;  // times the scale: -inf
    const lds_char* lds0 = (const lds_char*)smem;
    // the resident operands must have arrived before the loop, where the only vector-memory traffic
    // is the async tile loads and no compiler-placed wait may cover them
#pragma unroll
    for (int c = 0; c < CB; c++)
#pragma unroll
        for (int j = 0; j < NJ; j++) asm volatile("" ::"v"(kf[c].c[j]));

    // What the generated loop takes besides K: per-lane LDS addresses with everything wave-dependent folded in
    // (an LDS read of the loop is one of these registers plus a constant), the per-lane offsets of the tile
    // loads, and scalars.
    // (rows of 128 bytes: the two 16-row halves of a tile have transposed-operand addresses of their own)
    constexpr int NTR = OperandOffsets<E, D>::NS_TR;
    [[maybe_unused]] unsigned a_qrow[NJ], a_qtr[DB][NTR][2], a_vrow[NJ], a_vec = 0;
    if constexpr (kGen) {
        static_assert(L::kBlockAffine, "rows of 128 bytes and more");
        const unsigned ring = lds_address(smem + V_BYTES), vtile = lds_address(smem) + CB * wave * L::BLOCK_BYTES;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            a_qrow[j] = ring + ofs.row[j];
            a_vrow[j] = vtile + ofs.row[j];
        }
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int sx = 0; sx < NTR; sx++)
#pragma unroll
                for (int w = 0; w < 2; w++) a_qtr[db][sx][w] = ring + ofs.tr[db][sx][w];
        a_vec = ring + 2 * TILE_BYTES + 16 * h;
    }
    // first tile of iteration `it` and its pointers (the generated loop moves them on by itself)
    auto tile_pointers = [&](int it, const ET*& qp, const ET*& dop, const float*& lsep, const float*& delp) {
        const int g = it / n_tiles;
        const int q0 = (wg.start + it % n_tiles) * TQS;
        const int hq = hkv * p.group + g;
        qp = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hq * p.sq.h + (int64_t)q0 * p.sq.t;
        dop = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hq * p.sdo.h + (int64_t)q0 * p.sdo.t;
        lsep = p.lse + b * p.lse_b + hq * p.lse_h + q0;
        delp = p.delta + b * p.delta_b + hq * p.delta_h + q0;
    };
    // Iterations [it, it + n) that the generated loop may run for this wave: the wave's tiles are predicate-free,
    // and the tiles issued meanwhile (three ahead each) lie in the same query head and exist in full.  In the
    // last query head of the group the run may go on to the workgroup's last tile when all tiles exist in full:
    // its last iterations, which would request tiles past the end, take the loop's bodies that request nothing.
    const int run_first = imax(ta, fa);
    const int run_end = imin(imin(tb, fb), imin(n_tiles - (LA + 1), p.T / TQS - wg.start - (LA + 1)));
    const bool tail_ok = (wg.start + n_tiles) * TQS <= p.T;
    const int run_end_last = tail_ok ? imin(imin(tb, fb), n_tiles) : run_end;

    int st_cur = NS - 1;
    int st_issue = LA;
    int tile = -1;  // position of iteration `it` inside the q-tile range (it % n_tiles)
    for (int it = 0; it < n_iters; it++) {
        if constexpr (kGen) {
            const int t_next = tile + 1 == n_tiles ? 0 : tile + 1;
            const bool last_head = it >= n_iters - n_tiles;
            const int r_end = last_head ? run_end_last : run_end;
            int cnt = (t_next >= run_first) ? r_end - t_next : 0;
            // iterations of the run that would request a tile past the workgroup's last
            const unsigned tailn = uniform((unsigned)imax(0, r_end - (n_tiles - (LA + 1))));
            if (cnt >= 2 && p.scale_log2 != 0.f) {
                const ET *qp, *dop;
                const float *lsep, *delp;
                tile_pointers(it + LA + 1, qp, dop, lsep, delp);
                qp = uniform(qp), dop = uniform(dop), lsep = uniform(lsep), delp = uniform(delp);
                cnt = uniform(cnt);
                const int n_run = cnt;
                const unsigned st0 = uniform((unsigned)(st_cur + 1 == NS ? 0 : st_cur + 1));
                const unsigned ring = lds_address(smem + V_BYTES);
                const unsigned dmabase = uniform(ring + wave * 1024), vecdma = uniform(ring + 2 * TILE_BYTES);
                const unsigned qstep = uniform((unsigned)(TQS * p.sq.t * Elem<E>::kBytes));
                const unsigned dostep = uniform((unsigned)(TQS * p.sdo.t * Elem<E>::kBytes));
                const unsigned vecwave = uniform(wave == NW - 1 ? 1u : 0u);
                const unsigned lane4 = lane * 4;
                const float scale_s = uniform(p.scale_log2);
#define CHILL_DKDV_LOOP_ARGS_128                                                                                      \
    cnt, tok, qp, dop, lsep, delp, kf[0].c[0], kf[0].c[1], kf[0].c[2], kf[0].c[3], kf[0].c[4], kf[0].c[5], kf[0].c[6], \
        kf[0].c[7], kf[1].c[0], kf[1].c[1], kf[1].c[2], kf[1].c[3], kf[1].c[4], kf[1].c[5], kf[1].c[6], kf[1].c[7],     \
        a_qrow[0], a_qrow[1], a_qrow[2], a_qrow[3], a_qrow[4], a_qrow[5], a_qrow[6], a_qrow[7], a_qtr[0][0][0],         \
        a_qtr[0][0][1], a_qtr[1][0][0], a_qtr[1][0][1], a_qtr[2][0][0], a_qtr[2][0][1], a_qtr[3][0][0], a_qtr[3][0][1], \
        a_vrow[0], a_vrow[1], a_vrow[2], a_vrow[3], a_vrow[4], a_vrow[5], a_vrow[6], a_vrow[7], a_vec, load_q.goff[0],  \
        load_q.goff[1], load_do.goff[0], load_do.goff[1], lane4, scale_s, dmabase, vecdma, qstep, dostep, vecwave, st0, \
        tailn
#define CHILL_DKDV_LOOP_ARGS_64                                                                                       \
    cnt, tok, qp, dop, lsep, delp, kf[0].c[0], kf[0].c[1], kf[0].c[2], kf[0].c[3], kf[1].c[0], kf[1].c[1], kf[1].c[2], \
        kf[1].c[3], a_qrow[0], a_qrow[1], a_qrow[2], a_qrow[3], a_qtr[0][0][0], a_qtr[0][0][1], a_qtr[0][1][0],         \
        a_qtr[0][1][1], a_qtr[1][0][0], a_qtr[1][0][1], a_qtr[1][1][0], a_qtr[1][1][1], a_vrow[0], a_vrow[1],           \
        a_vrow[2], a_vrow[3], a_vec, load_q.goff[0], load_do.goff[0], lane4, scale_s, dmabase, vecdma, qstep, dostep,   \
        vecwave, st0, tailn
#define CHILL_DKDV_LOOP_CALL(loop, ...) loop(__VA_ARGS__)
                if constexpr (D == 128) {
                    if constexpr (std::is_same<E, bf16_t>::value) {
                        CHILL_DKDV_LOOP_CALL(CHILL_DKDV_LOOP_BF16_128, CHILL_DKDV_LOOP_ARGS_128);
                    } else {
                        CHILL_DKDV_LOOP_CALL(CHILL_DKDV_LOOP_F16_128, CHILL_DKDV_LOOP_ARGS_128);
                    }
                } else {
                    if constexpr (std::is_same<E, bf16_t>::value) {
                        CHILL_DKDV_LOOP_CALL(CHILL_DKDV_LOOP_BF16_64, CHILL_DKDV_LOOP_ARGS_64);
                    } else {
                        CHILL_DKDV_LOOP_CALL(CHILL_DKDV_LOOP_F16_64, CHILL_DKDV_LOOP_ARGS_64);
                    }
                }
#undef CHILL_DKDV_LOOP_CALL
#undef CHILL_DKDV_LOOP_ARGS_128
#undef CHILL_DKDV_LOOP_ARGS_64
                st_cur = (st_cur + n_run) % NS;
                st_issue = (st_issue + n_run) % NS;
                tile = t_next + n_run - 1;
                it += n_run - 1;
                continue;
            }
        }
        wait_async_tiles();
        __syncthreads();
        st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        tile = tile + 1 == n_tiles ? 0 : tile + 1;
        if (it + LA + 1 < n_iters) issue_iter(it + LA + 1, st_issue);
        if (tile < ta || tile >= tb) continue;
        const lds_char* q_tile = lds0 + V_BYTES + st_cur * STAGE_BYTES;
        const lds_char* do_tile = q_tile + TILE_BYTES;
        const lds_float* vec = reinterpret_cast<const lds_float*>(q_tile + 2 * TILE_BYTES);
        const bool full = (tile >= fa) && (tile < fb);
        const int q0 = (wg.start + tile) * TQS;

        f32x4 lse4[4], del4[4];
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++)
            lse4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + 8 * g4 + 4 * h);
        f32x16 s[CB], dp[CB];
        // S = Q K^T and dP = dO V^T, chunk by chunk: one Q (dO) chunk from LDS feeds all key blocks, and
        // consecutive MFMAs never write the same block
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const i32x4 aq = ofs.row_chunk(q_tile, 0, j, lane);
            const i32x4 ado = ofs.row_chunk(do_tile, 0, j, lane);
#pragma unroll
            for (int c = 0; c < CB; c++) {
                if (j == 0)
                    Mfma16<E>::set(aq, kf[c].c[j], s[c], tok);
                else
                    Mfma16<E>::add(aq, kf[c].c[j], s[c], tok);
            }
#pragma unroll
            for (int c = 0; c < CB; c++) {
                const i32x4 vc = ofs.row_chunk(lds0, CB * wave + c, j, lane);
                if (j == 0)
                    Mfma16<E>::set(ado, vc, dp[c], tok);
                else
                    Mfma16<E>::add(ado, vc, dp[c], tok);
            }
        }
        if constexpr (CB == 2)
            mfma_fence(s[0], s[1], dp[0], dp[1]);
        else
            mfma_fence(s[0], dp[0]);
        if (!full) {
#pragma unroll
            for (int c = 0; c < CB; c++) {
                const int k_pos = kw + 32 * c + n;
                if constexpr (Mask<MASK>::kRowIsRange) {
                    const Range vis = visible_range<MASK, false>(k_pos, seq_len, p.margs);
                    fill_outside_range(s[c], vis.lo, vis.hi, q0 + 4 * h, masked_score);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int q = q0 + 8 * (r / 4) + 4 * h + (r % 4);
                        const bool ok = (q < seq_len) && (k_pos < seq_len) && Mask<MASK>::pred(q, k_pos, seq_len, p.margs);
                        s[c][r] = ok ? s[c][r] : masked_score;
                    }
                }
            }
            // a row that attends to nothing has LSE2 = -inf and only masked entries
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float l = lse4[r / 4][r % 4];
                lse4[r / 4][r % 4] = (l == -INFINITY) ? 0.f : l;
            }
        }
#pragma unroll
        for (int c = 0; c < CB; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) s[c][r] = fast_exp2(__builtin_fmaf(s[c][r], scale, -lse4[r / 4][r % 4]));
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++)
            del4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + TQS + 8 * g4 + 4 * h);
        // dV^T += dO^T P: one transposed dO operand feeds all key blocks
        {
            i32x4 pb[CB][2];
#pragma unroll
            for (int c = 0; c < CB; c++) pack_block<E>(s[c], pb[c]);
            static_for<2>([&](auto sx) {
                static_for<DB>([&](auto db) {
                    const i32x4 a = ofs.tr_operand(do_tile, 0, sx, db, lane);
                    static_for<CB>([&](auto c) { Mfma16<E>::template acc<DV_BASE + 16 * (c * DB + db)>(a, pb[c][sx], tok); });
                });
            });
        }
        // dS = P (dP - delta); with V negated the chain has delivered -dP, and dS' = P (delta - dP) = -dS
#pragma unroll
        for (int c = 0; c < CB; c++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                dp[c][r] = kGen ? s[c][r] * (dp[c][r] + del4[r / 4][r % 4]) : s[c][r] * (dp[c][r] - del4[r / 4][r % 4]);
        // dK^T += Q^T dS
        {
            i32x4 sb[CB][2];
#pragma unroll
            for (int c = 0; c < CB; c++) pack_block<E>(dp[c], sb[c]);
            static_for<2>([&](auto sx) {
                static_for<DB>([&](auto db) {
                    const i32x4 a = ofs.tr_operand(q_tile, 0, sx, db, lane);
                    static_for<CB>([&](auto c) { Mfma16<E>::template acc<DK_BASE + 16 * (c * DB + db)>(a, sb[c][sx], tok); });
                });
            });
        }
    }

    agpr_drain(tok);
    static_for<CB>([&](auto c) {
        const int k_pos = kw + 32 * c + n;
        f32x16 acc[DB];
        const bool valid = k_pos < seq_len;
        static_for<DB>([&](auto db) { acc[db] = agpr_read_block<DK_BASE + 16 * (c * DB + db)>(); });
        if (k_pos < p.T)
            store_row_transposed<E, D>(dkbase + (int64_t)k_pos * p.sdk.t, acc, kGen ? -p.sm_scale : p.sm_scale, valid, h);
        static_for<DB>([&](auto db) { acc[db] = agpr_read_block<DV_BASE + 16 * (c * DB + db)>(); });
        if (k_pos < p.T) store_row_transposed<E, D>(dvbase + (int64_t)k_pos * p.sdv.t, acc, 1.f, valid, h);
    });
}

}  // namespace chill
