// dQ with the accumulators in hand-managed accumulation registers (16-bit inputs, wide rows).
//
// Same work split as dq_kernel (chill_bwd_kernels.h): a workgroup of 4 waves, one per SIMD, owns 128
// query rows, 32 per wave; a wave keeps its Q and dO rows in registers as MFMA B operands and streams
// K / V tiles of TK keys through the LDS ring (chill_bwd_dq.py:138-230).  At D = 256 the resident
// operands take 128 registers and the dQ^T accumulators another 128; left to the compiler, those
// accumulators travel between the two register files inside the loop (160 copies per 16 MFMAs).  Here
// they sit in the accumulation registers under fixed names (see the hand-placed MFMA helpers in
// chill_device.h) and only the 32 registers of the score blocks ever move.
//
//   S^T = K Q^T, dP^T = V dO^T, P = exp2(S * scale - LSE2), dS = P o (dP - delta),
//   dQ^T += K^T dS^T, finally dQ *= sm_scale                          (chill_bwd_dq.py:262-303, 171)
//
// Every translation unit that instantiates this kernel is checked (tests/test_abi.py) for the
// compiler keeping out of the accumulation registers the kernel names itself.
#pragma once

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"

namespace chill {

template <typename E, int D, int MASK, int TK, int NS>
__global__ __launch_bounds__(256) void dq_regs_kernel(BwdParams p, int n_q_tiles, int total_items,
                                                     int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    static_assert(Elem<E>::k16, "16-bit element types");
    constexpr int NW = 4;
    constexpr int TQ = NW * 32;
    constexpr int NT = NW * 64;
    constexpr int KB = TK / 32;
    constexpr int DB = (D + 31) / 32;
    constexpr int NJ = Resident<E, D>::NJ;
    constexpr int TILE_BYTES = LdsTile<E, D>::bytes(TK);
    constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K tile, then V tile
    constexpr int LA = NS - 2;
    static_assert(NS == 2 || NS == 3, "two or three LDS stages");
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
    auto issue_tile = [&](int i, int st_index) {
        int k0 = (wg.start + i) * TK;
        char* st = smem + st_index * STAGE_BYTES;
        load_k.issue(kptr + (int64_t)k0 * p.sk.t, p.T - k0, st, wave, lane);
        load_v.issue(vptr + (int64_t)k0 * p.sv.t, p.T - k0, st + TILE_BYTES, wave, lane);
    };
#pragma unroll
    for (int i = 0; i <= LA; i++)
        if (i < n_tiles) issue_tile(i, i);

    const int qw = qb + 32 * wave;
    const int q_pos = qw + n;
    OperandOffsets<E, D> ofs;
    ofs.init(lane);
    Resident<E, D> qf, dof;
    load_resident<E, D>(qf, qptr + (int64_t)qw * p.sq.t, p.sq.t, p.T - qw, lane);
    load_resident<E, D>(dof, doptr + (int64_t)qw * p.sdo.t, p.sdo.t, p.T - qw, lane);
    float lse_q = 0.f, delta_q = 0.f;
    if (q_pos < p.T) lse_q = p.lse[b * p.lse_b + hd * p.lse_h + q_pos];
    if (p.delta_out != nullptr) {
        const ET* optr = reinterpret_cast<const ET*>(p.o) + b * p.so.b + hd * p.so.h;
        delta_q = resident_row_delta<E, D>(dof, optr + (int64_t)qw * p.so.t, p.so.t, p.T - qw, lane);
        if (h == 0 && q_pos < p.T) p.delta_out[b * p.delta_b + hd * p.delta_h + q_pos] = delta_q;
    } else if (q_pos < p.T) {
        delta_q = p.delta[b * p.delta_b + hd * p.delta_h + q_pos];
    }
    // a row that attends to nothing has LSE2 = -inf and only masked entries (score -inf): P = exp2(-inf - 0)
    if (lse_q == -INFINITY) lse_q = 0.f;
    const Range vis = visible_range<MASK, true>(q_pos, seq_len, p.margs);  // the keys this lane's row sees

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    if (qw < seq_len) wr = tile_range<MASK, true>(qw, 32, TK, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    // accumulation registers: dQ^T block db at a[DQ_BASE + 16 * db], at the top of the file
    constexpr int DQ_BASE = 256 - 16 * DB;
    static_assert(DQ_BASE >= 0, "accumulators exceed the accumulation registers");
    agpr_reserve();
    int tok = agpr_zero<DQ_BASE, 16 * DB>();
    const float scale = p.scale_log2;
    const float masked_score = scale < 0.f ? INFINITY : -INFINITY;  // times the scale: -inf

    const lds_char* lds0 = (const lds_char*)smem;
    // the resident operands must have arrived before the loop, where the only vector-memory traffic
    // is the async tile loads and no compiler-placed wait may cover them
#pragma unroll
    for (int j = 0; j < NJ; j++) asm volatile("" ::"v"(qf.c[j]), "v"(dof.c[j]));
    asm volatile("" ::"v"(lse_q), "v"(delta_q));

    int st_cur = NS - 1;
    int st_issue = LA;
    for (int i = 0; i < n_tiles; i++) {
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
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            f32x16 cs, cdp;
            // S^T = K Q^T and dP^T = V dO^T, alternating so that consecutive MFMAs never write the same block
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const i32x4 ak = ofs.row_chunk(k_tile, kb, j, lane);
                const i32x4 av = ofs.row_chunk(v_tile, kb, j, lane);
                if (j == 0) {
                    Mfma16<E>::set(ak, qf.c[j], cs, tok);
                    Mfma16<E>::set(av, dof.c[j], cdp, tok);
                } else {
                    Mfma16<E>::add(ak, qf.c[j], cs, tok);
                    Mfma16<E>::add(av, dof.c[j], cdp, tok);
                }
            }
            mfma_fence(cs, cdp);
            if (!full) {
                if constexpr (Mask<MASK>::kRowIsRange) {
                    fill_outside_range(cs, vis.lo, vis.hi, k0 + 32 * kb + 4 * h, masked_score);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int k = k0 + 32 * kb + 8 * (r / 4) + 4 * h + (r % 4);
                        const bool ok = (q_pos < seq_len) && (k < seq_len) && Mask<MASK>::pred(q_pos, k, seq_len, p.margs);
                        cs[r] = ok ? cs[r] : masked_score;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float pv = fast_exp2(__builtin_fmaf(cs[r], scale, -lse_q));
                cdp[r] = pv * (cdp[r] - delta_q);
            }
            // dQ^T += K^T dS^T: one packed dS operand feeds all head-dim blocks
            i32x4 sb[2];
            pack_block<E>(cdp, sb);
            static_for<2>([&](auto sx) {
                static_for<DB>([&](auto db) {
                    const i32x4 a = ofs.tr_operand(k_tile, kb, sx, db, lane);
                    Mfma16<E>::template acc<DQ_BASE + 16 * db>(a, sb[sx], tok);
                });
            });
        }
    }

    agpr_drain(tok);
    f32x16 dq[DB];
    static_for<DB>([&](auto db) { dq[db] = agpr_read_block<DQ_BASE + 16 * db>(); });
    if (q_pos < p.T)
        store_row_transposed<E, D>(dqbase + (int64_t)q_pos * p.sdq.t, dq, p.sm_scale, q_pos < seq_len, h);
}

}  // namespace chill
