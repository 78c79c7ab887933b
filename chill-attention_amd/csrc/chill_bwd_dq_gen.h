// dQ with register-resident Q and dO, two 32-row query blocks per wave (16-bit inputs, head dim 128).
//
// A workgroup of 4 waves (one per SIMD, so each wave may use the whole 512-entry register file) owns
// 256 query rows, 64 per wave.  A wave keeps the Q and dO rows of its two blocks in the accumulation
// registers as MFMA B operands (128 registers) next to its dQ^T accumulators (2 x D/32 blocks, another
// 128), all under fixed names (see the hand-placed MFMA helpers in chill_device.h), and streams K / V
// tiles of 32 keys through a ring of four LDS stages (chill_bwd_dq.py:138-230): every K / V operand
// read from LDS feeds two MFMAs, half the LDS traffic per MFMA of dq_kernel.
//
//   S^T = K Q^T, dP^T = V dO^T, P = exp2(S * scale - LSE2), dS = P o (dP - delta),
//   dQ^T += K^T dS^T, finally dQ *= sm_scale                          (chill_bwd_dq.py:262-303, 171)
//
// Runs of tiles that are predicate-free for a wave's 64 rows go through a generated, software-pipelined
// loop (gen_dq_loop.py); the tiles under the mask are run by the code below, tile by tile.  Protocol of
// the ring, the same for both: the barrier of iteration i stands where a wave is done with tile i - 1
// and has seen its own loads of the tiles up to i + 1 land (the code below: at the top of iteration i;
// the generated loop: in the middle of its iteration i, which still reads tile i - 1 before); behind it
// the wave issues tile i + 3 into the stage of tile i - 1.  Tile 0 is certified by a barrier in front of
// the loop.
//
// Every translation unit that instantiates this kernel is checked (tests/test_abi.py) for the
// compiler keeping out of the accumulation registers the kernel names itself.
#pragma once

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"
#include "chill_dq_loop.inc"

// shortest run of predicate-free tiles that is handed to the generated loop
#ifndef CHILL_DQ_GEN_MIN_RUN
#define CHILL_DQ_GEN_MIN_RUN 2
#endif

namespace chill {

// a[BASE .. BASE + 3] = x (a resident MFMA operand)
template <int BASE>
__device__ __forceinline__ void agpr_write4(i32x4 x, int& tok) {
    asm("v_accvgpr_write_b32 a[%2], %1\n\tv_accvgpr_write_b32 a[%3], %4\n\tv_accvgpr_write_b32 a[%5], %6\n\tv_accvgpr_write_b32 a[%7], %8"
        : "+v"(tok)
        : "v"(x[0]), "n"(BASE), "n"(BASE + 1), "v"(x[1]), "n"(BASE + 2), "v"(x[2]), "n"(BASE + 3), "v"(x[3]));
}

// c = A B and c += A B with B = a[BREG .. BREG + 3] and c in ordinary registers
template <typename E>
struct Mfma16ResidentB;
#define CHILL_MFMA16_RB(TYPE, MNEMONIC)                                                                      \
    template <>                                                                                              \
    struct Mfma16ResidentB<TYPE> {                                                                           \
        template <int BREG>                                                                                  \
        __device__ __forceinline__ static void set(i32x4 a, f32x16& c, int& tok) {                           \
            asm(MNEMONIC " %0, %2, a[%3:%4], 0" : "=&v"(c), "+v"(tok) : "v"(a), "n"(BREG), "n"(BREG + 3));   \
        }                                                                                                    \
        template <int BREG>                                                                                  \
        __device__ __forceinline__ static void add(i32x4 a, f32x16& c, int& tok) {                           \
            asm(MNEMONIC " %0, %2, a[%3:%4], %0" : "+v"(c), "+v"(tok) : "v"(a), "n"(BREG), "n"(BREG + 3));   \
        }                                                                                                    \
    };
CHILL_MFMA16_RB(bf16_t, "v_mfma_f32_32x32x16_bf16")
CHILL_MFMA16_RB(f16_t, "v_mfma_f32_32x32x16_f16")
#undef CHILL_MFMA16_RB

template <typename E, int D, int MASK, int NS>
__global__ __launch_bounds__(256) void dq_regs2_kernel(BwdParams p, int n_q_tiles, int total_items,
                                                      int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    static_assert(Elem<E>::k16 && D == 128 && NS == 4, "16-bit inputs, head dim 128, four ring stages");
    typedef LdsTile<E, D> L;
    constexpr int NW = 4, CB = 2;
    constexpr int TQ = NW * CB * 32;
    constexpr int NT = NW * 64;
    constexpr int TK = 32;
    constexpr int DB = D / 32;
    constexpr int NJ = Resident<E, D>::NJ;
    constexpr int TILE_BYTES = L::bytes(TK);
    constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K tile, then V tile
    constexpr int LA = NS - 2;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int item = xcd_contiguous_item(blockIdx.x, total_items);
    if (item < 0) return;
    const int bh = item / n_q_tiles;
    const int qt = n_q_tiles - 1 - item % n_q_tiles;
    const int b = bh / p.H;
    const int hd = bh % p.H;
    const int hkv = hd / p.group;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;

    int seq_len = p.T;
    if (p.lens != nullptr) seq_len = imin(p.lens[(int64_t)b * p.lens_stride], p.T);

    const int qb = qt * TQ;
    ET* dqbase = reinterpret_cast<ET*>(p.dq) + b * p.sdq.b + hd * p.sdq.h;
    if (qb >= seq_len) {
        zero_rows<E, D, NT>(dqbase, p.sdq.t, qb, imin(TQ, p.T - qb), tid);
        if (p.delta_out != nullptr) {
            // (the dK/dV launch that follows reads delta of every row of the tiles it visits)
            for (int i = tid; i < imin(TQ, p.T - qb); i += NT) p.delta_out[b * p.delta_b + hd * p.delta_h + qb + i] = 0.f;
        }
        return;
    }

    const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h;
    const ET* doptr = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hd * p.sdo.h;
    const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
    const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;

    const TileRange wg = tile_range<MASK, true>(qb, TQ, TK, seq_len, false, p.margs);
    const int n_tiles = wg.end - wg.start;
    AsyncSwizzledLoader<E, D, TK, NT> load_k, load_v;
    load_k.init(p.sk.t, wave, lane);
    load_v.init(p.sv.t, wave, lane);
    static_assert(decltype(load_k)::PER_WAVE == 2, "two slabs of a tile per wave");
    auto issue_tile = [&](int i, int st_index) {
        int k0 = (wg.start + i) * TK;
        char* st = smem + st_index * STAGE_BYTES;
        load_k.issue(kptr + (int64_t)k0 * p.sk.t, p.T - k0, st, wave, lane);
        load_v.issue(vptr + (int64_t)k0 * p.sv.t, p.T - k0, st + TILE_BYTES, wave, lane);
    };
#pragma unroll
    for (int i = 0; i <= LA; i++)
        if (i < n_tiles) issue_tile(i, i);

    const int qw = qb + 32 * CB * wave;
    OperandOffsets<E, D> ofs;
    ofs.init(lane);

    // accumulation registers: dQ^T block (c, db) at a[16 * (c * DB + db)]; behind them Q chunk (c, j) at
    // a[Q_BASE + 4 * (c * NJ + j)] and dO chunk (c, j) at a[DO_BASE + 4 * (c * NJ + j)]
    constexpr int N_ACC = CB * DB * 16, Q_BASE = N_ACC, DO_BASE = Q_BASE + 4 * CB * NJ;
    static_assert(DO_BASE + 4 * CB * NJ == 256, "the accumulation registers are exactly taken");
    agpr_reserve();
    int tok = agpr_zero<0, N_ACC>();
    float lse_q[CB], delta_q[CB];
    f32x16 neg_delta[CB];   // what the dP'^T chains of the generated loop start from
    static_for<CB>([&](auto c) {
        const int q0 = qw + 32 * c;
        Resident<E, D> qf, dof;
        load_resident<E, D>(qf, qptr + (int64_t)q0 * p.sq.t, p.sq.t, p.T - q0, lane);
        load_resident<E, D>(dof, doptr + (int64_t)q0 * p.sdo.t, p.sdo.t, p.T - q0, lane);
        lse_q[c] = 0.f;
        delta_q[c] = 0.f;
        if (q0 + n < p.T) lse_q[c] = p.lse[b * p.lse_b + hd * p.lse_h + q0 + n];
        if (p.delta_out != nullptr) {
            const ET* optr = reinterpret_cast<const ET*>(p.o) + b * p.so.b + hd * p.so.h;
            delta_q[c] = resident_row_delta<E, D>(dof, optr + (int64_t)q0 * p.so.t, p.so.t, p.T - q0, lane);
            if (h == 0 && q0 + n < p.T) p.delta_out[b * p.delta_b + hd * p.delta_h + q0 + n] = delta_q[c];
        } else if (q0 + n < p.T) {
            delta_q[c] = p.delta[b * p.delta_b + hd * p.delta_h + q0 + n];
        }
        // a row that attends to nothing has LSE2 = -inf and only masked entries (score -inf): P = exp2(-inf - 0)
        if (lse_q[c] == -INFINITY) lse_q[c] = 0.f;
        static_for<NJ>([&](auto j) {
            agpr_write4<Q_BASE + 4 * (c * NJ + j)>(qf.c[j], tok);
            agpr_write4<DO_BASE + 4 * (c * NJ + j)>(dof.c[j], tok);
        });
#pragma unroll
        for (int r = 0; r < 16; r++) neg_delta[c][r] = -delta_q[c];
        asm volatile("" : "+v"(neg_delta[c]));
    });

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    // (rows of the wave at and beyond seq_len are computed like the others and never stored)
    if (qw < seq_len) wr = tile_range_rows_discarded<MASK, true>(qw, 32 * CB, TK, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    const float scale = p.scale_log2;
    const float masked_score = scale < 0.f ? INFINITY : -INFINITY;  // times the scale: -inf
    const lds_char* lds0 = (const lds_char*)smem;

    // what the generated loop takes: per-lane LDS addresses (a read of the loop is one of them plus a constant)
    static_assert(L::kBlockAffine && OperandOffsets<E, D>::kHalfAffine, "rows of 256 bytes");
    unsigned a_krow[NJ], a_ktr[DB][2];
#pragma unroll
    for (int j = 0; j < NJ; j++) a_krow[j] = lds_address(smem) + ofs.row[j];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int w = 0; w < 2; w++) a_ktr[db][w] = lds_address(smem) + ofs.tr[db][0][w];
    // iterations [i, run_end) may go through the generated loop if i >= run_first: the wave's 64 rows see every key
    // of those tiles, and the tiles issued meanwhile (three ahead each) exist in full
    const int run_first = imax(ta, fa);
    const int run_end = imin(imin(tb, fb), imin(n_tiles - (LA + 1), p.T / TK - wg.start - (LA + 1)));

    // tile 0 has landed for everyone (the barrier of iteration i certifies the tiles up to i + 1 only)
    wait_async_tiles();
    __syncthreads();

    int st_cur = NS - 1;
    int st_issue = LA;
    for (int i = 0; i < n_tiles; i++) {
        {
            int cnt = (i >= run_first) ? run_end - i : 0;
            if (cnt >= CHILL_DQ_GEN_MIN_RUN && scale != 0.f) {
                cnt = uniform(cnt);
                const int n_run = cnt;
                const ET* kp = uniform(kptr + (int64_t)(wg.start + i + LA + 1) * TK * p.sk.t);
                const ET* vp = uniform(vptr + (int64_t)(wg.start + i + LA + 1) * TK * p.sv.t);
                const unsigned st0 = uniform((unsigned)(st_cur + 1 == NS ? 0 : st_cur + 1));
                const unsigned dmabase = uniform(lds_address(smem) + wave * 1024);
                const unsigned kstep = uniform((unsigned)(TK * p.sk.t * Elem<E>::kBytes));
                const unsigned vstep = uniform((unsigned)(TK * p.sv.t * Elem<E>::kBytes));
                const float scale_s = uniform(scale);
#define CHILL_DQ_LOOP_ARGS                                                                                              \
    cnt, tok, kp, vp, neg_delta[0], neg_delta[1], lse_q[0], lse_q[1], a_krow[0], a_krow[1], a_krow[2], a_krow[3], a_krow[4], \
        a_krow[5], a_krow[6], a_krow[7], a_ktr[0][0], a_ktr[0][1], a_ktr[1][0], a_ktr[1][1], a_ktr[2][0], a_ktr[2][1],     \
        a_ktr[3][0], a_ktr[3][1], load_k.goff[0], load_k.goff[1], load_v.goff[0], load_v.goff[1], scale_s, dmabase, kstep, \
        vstep, st0
#define CHILL_DQ_LOOP_CALL(loop, ...) loop(__VA_ARGS__)
                if constexpr (std::is_same<E, bf16_t>::value) {
                    CHILL_DQ_LOOP_CALL(CHILL_DQ_LOOP_BF16_128, CHILL_DQ_LOOP_ARGS);
                } else {
                    CHILL_DQ_LOOP_CALL(CHILL_DQ_LOOP_F16_128, CHILL_DQ_LOOP_ARGS);
                }
#undef CHILL_DQ_LOOP_CALL
#undef CHILL_DQ_LOOP_ARGS
                st_cur = (st_cur + n_run) % NS;
                st_issue = (st_issue + n_run) % NS;
                i += n_run - 1;
                continue;
            }
        }
        wait_async_tiles();
        __syncthreads();
        st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        if (i + LA + 1 < n_tiles) issue_tile(i + LA + 1, st_issue);
        if (i < ta || i >= tb) continue;
        const lds_char* k_tile = lds0 + st_cur * STAGE_BYTES;
        const lds_char* v_tile = k_tile + TILE_BYTES;
        const bool full = (i >= fa) && (i < fb);
        const int k0 = (wg.start + i) * TK;
        f32x16 cs[CB], cdp[CB];
        // S^T = K Q^T and dP^T = V dO^T: one K (V) chunk from LDS feeds both query blocks
        static_for<NJ>([&](auto j) {
            const i32x4 ak = ofs.row_chunk(k_tile, 0, j, lane);
            const i32x4 av = ofs.row_chunk(v_tile, 0, j, lane);
            static_for<CB>([&](auto c) {
                if constexpr (j == 0) {
                    Mfma16ResidentB<E>::template set<Q_BASE + 4 * (c * NJ + j)>(ak, cs[c], tok);
                    Mfma16ResidentB<E>::template set<DO_BASE + 4 * (c * NJ + j)>(av, cdp[c], tok);
                } else {
                    Mfma16ResidentB<E>::template add<Q_BASE + 4 * (c * NJ + j)>(ak, cs[c], tok);
                    Mfma16ResidentB<E>::template add<DO_BASE + 4 * (c * NJ + j)>(av, cdp[c], tok);
                }
            });
        });
        mfma_fence(cs[0], cs[1], cdp[0], cdp[1]);
        i32x4 sb[CB][2];
#pragma unroll
        for (int c = 0; c < CB; c++) {
            const int q_pos = qw + 32 * c + n;
            if (!full) {
                if constexpr (Mask<MASK>::kRowIsRange) {
                    const Range vis = visible_range<MASK, true>(q_pos, seq_len, p.margs);
                    fill_outside_range(cs[c], vis.lo, vis.hi, k0 + 4 * h, masked_score);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int k = k0 + 8 * (r / 4) + 4 * h + (r % 4);
                        const bool ok = (q_pos < seq_len) && (k < seq_len) && Mask<MASK>::pred(q_pos, k, seq_len, p.margs);
                        cs[c][r] = ok ? cs[c][r] : masked_score;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float pv = fast_exp2(__builtin_fmaf(cs[c][r], scale, -lse_q[c]));
                cdp[c][r] = pv * (cdp[c][r] - delta_q[c]);
            }
            pack_block<E>(cdp[c], sb[c]);
        }
        // dQ^T += K^T dS^T: one transposed K operand feeds both query blocks
        static_for<2>([&](auto sx) {
            static_for<DB>([&](auto db) {
                const i32x4 a = ofs.tr_operand(k_tile, 0, sx, db, lane);
                static_for<CB>([&](auto c) { Mfma16<E>::template acc<16 * (c * DB + db)>(a, sb[c][sx], tok); });
            });
        });
    }

    agpr_drain(tok);
    static_for<CB>([&](auto c) {
        const int q_pos = qw + 32 * c + n;
        f32x16 dq[DB];
        static_for<DB>([&](auto db) { dq[db] = agpr_read_block<16 * (c * DB + db)>(); });
        if (q_pos < p.T) store_row_transposed<E, D>(dqbase + (int64_t)q_pos * p.sdq.t, dq, p.sm_scale, q_pos < seq_len, h);
    });
}

}  // namespace chill
