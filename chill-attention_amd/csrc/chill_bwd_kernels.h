// Backward kernels: delta = rowsum(O * dO), dQ, and dK/dV — the gfx950 counterparts of the
// reference's _chill_attn_bwd_precompute (chill_attention/utils.py:94-217), _chill_attn_bwd_dq
// (chill_bwd_dq.py:15-397) and _chill_attn_bwd_dkdv (chill_bwd_dkdv.py:15-509).
//
// Both matrix kernels use the building blocks of the forward: a wave owns 32 resident rows whose
// operands sit in registers as MFMA B operands; the streamed tiles sit in LDS and are read both
// row-wise (products with the resident rows) and through the transposing read (products that
// accumulate INTO the resident rows).  All accumulators are transposed ([head dim][resident row]),
// so every per-row quantity is a per-lane scalar.
//
//   dQ   (resident: Q, dO rows; streamed: K, V tiles)
//        S^T = K Q^T, dP^T = V dO^T, P^T = exp2(S^T * scale - LSE2), dS^T = P^T o (dP^T - delta),
//        dQ^T += K^T dS^T, finally dQ *= sm_scale                      (chill_bwd_dq.py:312-332, 396)
//   dKdV (resident: K, V rows; streamed: Q, dO tiles with their LSE2 / delta)
//        S = Q K^T, dP = dO V^T, P, dS as above,
//        dV^T += dO^T P, dK^T += Q^T dS, finally dK *= sm_scale        (chill_bwd_dkdv.py:362-403, 230)
#pragma once

#include <type_traits>

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"
#include "chill_bwd_dkdv_regs.h"
#include "chill_bwd_dq_regs.h"
#include "chill_bwd_dq_gen.h"

namespace chill {

// ------------------------------------------------------------------------------------------ delta
// One 16-byte chunk of O and of dO per thread and step; the CH lanes that share a row reduce with
// butterfly shuffles.  Pure streaming: 2 * D * es bytes read and 4 bytes written per row.
template <typename E, int D>
__global__ __launch_bounds__(256) void delta_kernel(DeltaParams p) {
    using ET = typename Elem<E>::type;
    constexpr int CH = LdsTile<E, D>::CH;      // lanes per row (2 .. 64)
    constexpr int EPC = 16 / Elem<E>::kBytes;  // elements per chunk
    constexpr int ROWS_PER_STEP = 256 / CH;
    constexpr int STEPS = 4;
    const int b = blockIdx.z, hd = blockIdx.y;
    const ET* obase = reinterpret_cast<const ET*>(p.o) + b * p.so.b + hd * p.so.h;
    const ET* dobase = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hd * p.sdo.h;
    float* dbase = p.delta + b * p.delta_b + hd * p.delta_h;
    const int c = threadIdx.x % CH;
    const int rsub = threadIdx.x / CH;
    const int row0 = blockIdx.x * (ROWS_PER_STEP * STEPS);
    i32x4 ov[STEPS], dv[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        int row = row0 + s * ROWS_PER_STEP + rsub;
        ov[s] = i32x4{0, 0, 0, 0};
        dv[s] = i32x4{0, 0, 0, 0};
        if (row < p.T) {
            ov[s] = *reinterpret_cast<const i32x4*>(reinterpret_cast<const char*>(obase + (int64_t)row * p.so.t) + c * 16);
            dv[s] = *reinterpret_cast<const i32x4*>(reinterpret_cast<const char*>(dobase + (int64_t)row * p.sdo.t) + c * 16);
        }
    }
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
        int row = row0 + s * ROWS_PER_STEP + rsub;
        const ET* oe = reinterpret_cast<const ET*>(&ov[s]);
        const ET* de = reinterpret_cast<const ET*>(&dv[s]);
        float acc = 0.f;
#pragma unroll
        for (int e = 0; e < EPC; e++) acc += Elem<E>::to_float(oe[e]) * Elem<E>::to_float(de[e]);
#pragma unroll
        for (int off = CH / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (c == 0 && row < p.T) dbase[row] = acc;
    }
}

template <typename E, int D>
int launch_delta(const DeltaParams& p, hipStream_t stream) {
    constexpr int CH = LdsTile<E, D>::CH;
    constexpr int ROWS_PER_BLOCK = (256 / CH) * 4;
    dim3 grid(cdiv(p.T, ROWS_PER_BLOCK), p.H, p.B), block(256);
    if (p.H > 65535 || p.B > 65535) return CHILL_ERR_TOO_LARGE;
    hipLaunchKernelGGL((delta_kernel<E, D>), grid, block, 0, stream, p);
    return hipGetLastError() == hipSuccess ? CHILL_OK : CHILL_ERR_HIP;
}

// Probabilities and score gradients of one 32x32 block, in place: on entry s = raw scores,
// dp = dO.V products; on exit s = P (0 where masked), dp = dS = P * (dP - delta).  A row that saw
// no key has LSE2 = -inf and P = exp2(+inf) = inf there; such a row can only occur in blocks that
// take the predicate path, whose select (not a multiply) turns it into 0.
// Row/column meaning differs between the two kernels, so the caller supplies, per accumulator
// register r, the LSE2 / delta of the query and the (q, k) positions.
template <int MASK, bool PARTIAL, typename PosFn>
__device__ __forceinline__ void softmax_grad_block(f32x16& s, f32x16& dp, float scale, int seq_len,
                                                   MaskArgs a, PosFn pos) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
        int q, k;
        float lse, delta;
        pos(r, q, k, lse, delta);
        float pv = fast_exp2(s[r] * scale - lse);
        if (PARTIAL) {
            bool ok = (q < seq_len) && (k < seq_len) && Mask<MASK>::pred(q, k, seq_len, a);
            pv = ok ? pv : 0.f;
        }
        s[r] = pv;
        dp[r] = pv * (dp[r] - delta);
    }
}

}  // namespace chill
#include "chill_bwd_small.h"
namespace chill {

// ------------------------------------------------------------------------------------------ dQ
// Same skeleton as the forward kernel: asynchronous K/V ring, 32-key steps, the two score GEMMs of
// step t+1 (S^T and dP^T) issued before the vector work of step t.
// Workgroups of four waves whose LDS ring leaves room for a second workgroup on the CU are compiled
// for 256 registers per wave, so that two of them share a CU: one computes while the other loads its
// first tiles or stores its result.
template <typename E, int D, int NW, int TK, int NS>
constexpr int dq_waves_per_simd() {
    return (NW == 4 && Elem<E>::k16 && 2 * NS * 2 * LdsTile<E, D>::bytes(TK) <= 160 * 1024) ? 2 : 1;
}

template <typename E, int D, int MASK, int NW, int TK, int NS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(dq_waves_per_simd<E, D, NW, TK, NS>())))
void dq_kernel(BwdParams p, int n_q_tiles, int total_items,
                                                     int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
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

    const int item = xcd_contiguous_item(blockIdx.x, total_items, dq_waves_per_simd<E, D, NW, TK, NS>());
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

    f32x16 dq[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) dq[i][r] = 0.f;
    const float scale = p.scale_log2;
    const float masked_score = scale < 0.f ? INFINITY : -INFINITY;  // times the scale: -inf

    // S^T = K Q^T and dP^T = V dO^T of step kb of the stage at `stage`
    auto gemms = [&](f32x16& sdst, f32x16& dpdst, const lds_char* stage, int kb) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            sdst[r] = 0.f;
            dpdst[r] = 0.f;
        }
        sdst = mma_rowwise<E, D>(stage, kb, ofs, qf, sdst, lane);
        dpdst = mma_rowwise<E, D>(stage + TILE_BYTES, kb, ofs, dof, dpdst, lane);
    };

    const lds_char* lds0 = (const lds_char*)smem;
    // the resident operands must have arrived before the loop, where the only vector-memory traffic
    // is the async tile loads and no compiler-placed wait may cover them
#pragma unroll
    for (int j = 0; j < NJ; j++) asm volatile("" ::"v"(qf.c[j]), "v"(dof.c[j]));
    asm volatile("" ::"v"(lse_q), "v"(delta_q));

    typedef LdsTile<E, D> L;
    constexpr bool kFold = L::kBlockAffine && Elem<E>::k16;
    if constexpr (kFold) {
        // Block-affine 16-bit tiles: the loop is unrolled over the ring stages and every LDS read is a
        // loop-invariant per-lane pointer plus a constant in the instruction's offset field.  S^T and dP^T
        // of a 32-key step are one chain of 2 NJ MFMAs whose operands are read kPrefetch steps ahead, in
        // this order and no other (left to itself the compiler reads each operand right before its MFMA
        // and the wave waits out the LDS latency 2 NJ times per step); the exponentials are spread over
        // the dP^T half of the chain.
        constexpr int kPrefetch = 4;  // C3: 2.95 ms in the compiler's order, 2.80 with 3 (then 2.84 -> 2.79 with delta in the
                                      // accumulators, 2.76 with 4)
        OperandPointers<E, D> at;
        at.template init<true>(ofs, lds0);
        // dP^T - delta comes out of the MFMA chain itself: its accumulators start at -delta (the lane's
        // query row has one delta), which saves a subtraction per entry
        f32x16 neg_delta;
#pragma unroll
        for (int r = 0; r < 16; r++) neg_delta[r] = -delta_q;
        asm volatile("" : "+v"(neg_delta));
        auto tile_step = [&](auto st_tag, int i) {
            constexpr int ST = decltype(st_tag)::value;
            wait_async_tiles();
            __syncthreads();
            if (i + LA + 1 < n_tiles) issue_tile(i + LA + 1, (ST + NS - 1) % NS);
            if (i < ta || i >= tb) return;
            const bool full = (i >= fa) && (i < fb);
            const int k0 = (wg.start + i) * TK;
            static_for<KB>([&](auto kb) {
                constexpr int K_AT = ST * STAGE_BYTES + kb * L::BLOCK_BYTES, V_AT = K_AT + TILE_BYTES;
                f32x16 cs, cdp;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    cs[r] = 0.f;
                    cdp[r] = neg_delta[r];
                }
                i32x4 op[2 * NJ];
                auto fetch = [&](auto t_tag) {
                    constexpr int t = decltype(t_tag)::value;
                    if constexpr (t < NJ) {
                        op[t] = at.row_chunk(K_AT, t);
                    } else if constexpr (t < 2 * NJ) {
                        op[t] = at.row_chunk(V_AT, t - NJ);
                    }
                };
                static_for<kPrefetch>([&](auto t) { fetch(t); });
                __builtin_amdgcn_sched_barrier(0);
                static_for<NJ>([&](auto t) {
                    cs = Elem<E>::mma(op[t], qf.c[t], cs);
                    asm volatile("" : "+v"(cs));  // keeps the MFMA at this place of the chain
                    fetch(std::integral_constant<int, t + kPrefetch>{});
                    __builtin_amdgcn_sched_barrier(0);
                });
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
                constexpr int PER = (16 + NJ - 1) / NJ;  // exponentials per step
                static_for<NJ>([&](auto t) {
                    cdp = Elem<E>::mma(op[NJ + t], dof.c[t], cdp);
                    asm volatile("" : "+v"(cdp));
                    fetch(std::integral_constant<int, NJ + t + kPrefetch>{});
#pragma unroll
                    for (int r = PER * t; r < PER * (t + 1) && r < 16; r++)
                        cs[r] = fast_exp2(__builtin_fmaf(cs[r], scale, -lse_q));
                    // the last steps stay open to what follows: the first operands of dQ^T are read behind them
                    if constexpr (t + 2 < NJ) __builtin_amdgcn_sched_barrier(0);
                });
#pragma unroll
                for (int r = 0; r < 16; r++) cdp[r] = cs[r] * cdp[r];
                mma_transposed<E, D>(K_AT, at, cdp, dq);  // dQ^T += K^T dS^T
            });
        };
        for (int i = 0; i < n_tiles; i += NS)
            static_for<NS>([&](auto st) {
                if (i + st < n_tiles) tile_step(st, i + st);
            });
    } else {
        int st_cur = NS - 1;
        int st_issue = LA;
        for (int i = 0; i < n_tiles; i++) {
            wait_async_tiles();
            __syncthreads();
            st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
            st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
            if (i + LA + 1 < n_tiles) issue_tile(i + LA + 1, st_issue);
            if (i < ta || i >= tb) continue;
            const lds_char* stage = lds0 + st_cur * STAGE_BYTES;
            const bool full = (i >= fa) && (i < fb);
            const int k0 = (wg.start + i) * TK;
            // Masked entries get a score of -inf (times the sign of the scale) in a branch of their own, so that
            // the rest of the tile is the same straight-line code for full and partial tiles, in which the
            // compiler places the vector work of one 32-key step among the MFMAs of the next.
    #pragma unroll
            for (int kb = 0; kb < KB; kb++) {
                f32x16 cs, cdp;
                gemms(cs, cdp, stage, kb);
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
                // dQ^T += K^T dS^T
                mma_transposed<E, D>(stage, kb, ofs, cdp, dq, lane);
            }
        }

    }

    if (q_pos < p.T)
        store_row_transposed<E, D>(dqbase + (int64_t)q_pos * p.sdq.t, dq, p.sm_scale, q_pos < seq_len, h);
}

// One (mask, tile shape): SHORT selects the table row for short sequences.
// (defined below, next to the kernel it is modelled on)
template <typename E, int D, int MASK, int NW, int NS>
__global__ void dq_split_kernel(BwdParams p, int n_q_tiles, int total_items, int wave_has_full_blocks);

template <typename E, int D, int MASK_ID, bool SHORT>
int launch_dq_shape(const BwdParams& p, hipStream_t stream) {
    constexpr int kRowFor = SHORT ? 1 : kLongSequence;
    constexpr TileConfig cfg = dq_tile_config(MASK_ID, D, Elem<E>::kDType, kRowFor);
    static_assert(cfg.rows == cfg.waves * (dq_is_split(D, Elem<E>::kDType) ? 16 : 32), "one wave (or a pair) owns 32 rows");
    constexpr int NS = dq_stages(MASK_ID, D, Elem<E>::kDType, kRowFor);
    const int n_q_tiles = cdiv(p.T, cfg.rows);
    const int64_t total64 = (int64_t)p.B * p.H * n_q_tiles;
    if (total64 > ((int64_t)1 << 30)) return CHILL_ERR_TOO_LARGE;
    const int total = (int)total64;
    dim3 grid(cdiv(total, 8) * 8), block(cfg.waves * 64);
    void (*kern)(BwdParams, int, int, int);
    if constexpr (dq_regs_keys(D, Elem<E>::kDType) > 0)
        kern = dq_regs_kernel<E, D, MASK_ID, cfg.streamed, NS>;
    else if constexpr (dq_is_split(D, Elem<E>::kDType))
        kern = dq_split_kernel<E, D, MASK_ID, cfg.waves, NS>;
    else
        kern = dq_kernel<E, D, MASK_ID, cfg.waves, cfg.streamed, NS>;
    const bool hfb = Mask<MASK_ID>::has_full_blocks(32, cfg.streamed, p.T, p.margs);
    if (cfg.lds_bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                cfg.lds_bytes) != hipSuccess)
            return CHILL_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, grid, block, cfg.lds_bytes, stream, p, n_q_tiles, total, hfb ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

// dQ with register-resident Q and dO (16-bit inputs at head dim 128, long sequences on full grids)
template <typename E, int D, int MASK_ID>
int launch_dq_regs2(const BwdParams& p, hipStream_t stream) {
    constexpr TileConfig cfg = dq_regs2_tile_config(D, Elem<E>::kDType);
    const int n_q_tiles = cdiv(p.T, cfg.rows);
    const int64_t total64 = (int64_t)p.B * p.H * n_q_tiles;
    if (total64 > ((int64_t)1 << 30)) return CHILL_ERR_TOO_LARGE;
    const int total = (int)total64;
    void (*kern)(BwdParams, int, int, int) = dq_regs2_kernel<E, D, MASK_ID, 4>;
    const bool hfb = Mask<MASK_ID>::has_full_blocks(64, cfg.streamed, p.T, p.margs);
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, cfg.lds_bytes) !=
        hipSuccess)
        return CHILL_ERR_HIP;
    hipLaunchKernelGGL(kern, dim3(cdiv(total, 8) * 8), dim3(cfg.waves * 64), cfg.lds_bytes, stream, p, n_q_tiles, total, hfb ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

// A launch far too small for the chip: 32 rows per workgroup, the streamed axis split over its waves.
// PASS 1: dQ (workgroups over query blocks), 2: dK/dV (over key blocks).
template <typename E, int D, int MASK_ID, int PASS>
int launch_bwd_small(const BwdParams& p, hipStream_t stream) {
    constexpr int kLdsOne = bwd_small_lds_bytes(D, Elem<E>::kDType, PASS);
    const int n_tiles = cdiv(p.T, 32);
    const long long heads = (long long)p.B * (PASS == 1 ? p.H : p.H_kv);  // (few by bwd_takes_small)
    // (dK/dV keeps one block per workgroup: with K, V and two accumulators a wave needs more than the 256 registers it
    // would be left with)
    constexpr bool kTwoFit = PASS == 1 && small_fits_two_tiles(kLdsOne);
    bool two = false;
    if constexpr (kTwoFit) two = small_takes_two_tiles(heads * n_tiles);
    const int total = (int)(heads * (two ? (n_tiles + 1) / 2 : n_tiles));
    const int lds_bytes = two ? 2 * kLdsOne : kLdsOne;
    void (*kern)(BwdParams, int, int, int);
    if constexpr (PASS == 1)
        kern = dq_small_kernel<E, D, MASK_ID, 1>;
    else
        kern = dkdv_small_kernel<E, D, MASK_ID>;
    if constexpr (kTwoFit) {
        if (two) kern = dq_small_kernel<E, D, MASK_ID, 2>;
    }
    const bool hfb = Mask<MASK_ID>::has_full_blocks(32, 32, p.T, p.margs);
    if (lds_bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds_bytes) != hipSuccess)
            return CHILL_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, dim3(total), dim3(kFwdSmallWaves * 64 * (two ? 2 : 1)), lds_bytes, stream, p, n_tiles, total,
                       hfb ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

template <typename E, int D>
int launch_dq(const BwdParams& p, int mask_id, hipStream_t stream) {
    const int64_t max_stride = p.sk.t > p.sv.t ? p.sk.t : p.sv.t;
    if (max_stride * Elem<E>::kBytes * 256 >= ((int64_t)1 << 31)) return CHILL_ERR_TOO_LARGE;
    int status = CHILL_ERR_BAD_MASK;
    CHILL_DISPATCH_MASK(mask_id, {
        // the table has a row of its own for short sequences and small grids where that row differs
        constexpr bool has_short_row = dq_tile_config(MASK_ID, D, Elem<E>::kDType, 1).waves !=
                                       dq_tile_config(MASK_ID, D, Elem<E>::kDType).waves;
        bool small = false;
        constexpr bool served = bwd_small_serves(D, Elem<E>::kDType, CHILL_PASS_DQ);
        if constexpr (served) small = bwd_takes_small(MASK_ID, (long long)p.B * p.H, p.T, D, Elem<E>::kDType, CHILL_PASS_DQ);
        bool regs2 = false;
        if constexpr (dq_regs2_is_optional(D, Elem<E>::kDType)) regs2 = dq_takes_regs2(MASK_ID, (long long)p.B * p.H, p.T);
        if (small) {
            if constexpr (served) status = launch_bwd_small<E, D, MASK_ID, 1>(p, stream);
        } else if (regs2) {
            if constexpr (dq_regs2_is_optional(D, Elem<E>::kDType)) status = launch_dq_regs2<E, D, MASK_ID>(p, stream);
        } else if constexpr (has_short_row) {
            status = dq_takes_short_row((long long)p.B * p.H, p.T) ? launch_dq_shape<E, D, MASK_ID, true>(p, stream)
                                                                   : launch_dq_shape<E, D, MASK_ID, false>(p, stream);
        } else {
            status = launch_dq_shape<E, D, MASK_ID, false>(p, stream);
        }
    });
    return status;
}

// ------------------------------------------------------------------------------------------ dQ (wide rows)
// fp32 rows of 1 KiB (head dim 256): a wave that owns 32 query rows would hold Q and dO as resident
// operands (256 registers) and dQ^T (128): dq_kernel spilled 245 registers there.  Two waves share a
// 32-query block instead, the way dkdv_split_kernel's waves share a key block: the even one holds Q and
// computes S^T = K Q^T (scale and LSE2 applied), the odd one holds dO and computes dP^T = V dO^T - delta;
// the two products meet in LDS, both waves compute P and dS, and each accumulates half of the head-dim
// blocks of dQ^T += K^T dS^T.  No MFMA is issued twice and both waves issue the same number.
template <typename E, int D, int MASK, int NW, int NS>
__global__ __launch_bounds__(NW * 64) void dq_split_kernel(BwdParams p, int n_q_tiles, int total_items,
                                                      int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    typedef LdsTile<E, D> L;
    static_assert(!Elem<E>::k16, "fp32 rows");
    constexpr int TK = 32;
    constexpr int NQB = NW / 2;       // 32-query blocks per workgroup
    constexpr int TQ = NQB * 32;
    constexpr int NT = NW * 64;
    constexpr int DB = D / 32;
    constexpr int DBW = DB / 2;       // head-dim blocks a wave accumulates
    constexpr int NJ = L::CH / 2;
    constexpr int TILE_BYTES = L::bytes(TK);
    constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K tile, then V tile
    constexpr int X_BYTES = 16 * 64 * 4;         // one product
    static_assert(NS == 2, "two ring stages");
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
    const int qblk = wave % NQB;
    const int role = wave / NQB;  // 0: S from Q, 1: dP from dO; also the half of the head dim it accumulates
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
    if (n_tiles > 0) issue_tile(0, 0);

    // this wave's resident operand: the block's Q rows (role 0) or dO rows (role 1); LSE2 or delta of
    // the lane's row
    const int qw = qb + 32 * qblk;
    const int q_pos = qw + n;
    Resident<E, D> res;
    float sub = 0.f;
    {
        const int64_t stride = role == 0 ? p.sq.t : p.sdo.t;
        const ET* src = role == 0 ? reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hd * p.sq.h
                                  : reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hd * p.sdo.h;
        load_resident<E, D>(res, src + (int64_t)qw * stride, stride, p.T - qw, lane);
        if (role == 1 && p.delta_out != nullptr) {
            const ET* optr = reinterpret_cast<const ET*>(p.o) + b * p.so.b + hd * p.so.h;
            sub = resident_row_delta<E, D>(res, optr + (int64_t)qw * p.so.t, p.so.t, p.T - qw, lane);
            if (h == 0 && q_pos < p.T) p.delta_out[b * p.delta_b + hd * p.delta_h + q_pos] = sub;
        } else if (q_pos < p.T) {
            sub = role == 0 ? p.lse[b * p.lse_b + hd * p.lse_h + q_pos] : p.delta[b * p.delta_b + hd * p.delta_h + q_pos];
        }
        // a row that attends to nothing has LSE2 = -inf and only masked entries, which a select zeroes
        if (role == 0 && sub == -INFINITY) sub = 0.f;
    }

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    if (qw < seq_len) wr = tile_range<MASK, true>(qw, 32, TK, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    f32x16 dq[DBW];
#pragma unroll
    for (int i = 0; i < DBW; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) dq[i][r] = 0.f;
    const float mult = role == 0 ? p.scale_log2 : 1.f;
    const lds_char* lds0 = (const lds_char*)smem;
    // the two products of block qblk: register r of lane l at ((r / 4) * 64 + l) * 16 + (r % 4) * 4
    char* xblock = smem + 2 * STAGE_BYTES + qblk * 2 * X_BYTES;
    const int db0 = role * DBW;

    for (int it = 0; it < n_tiles; it++) {
        wait_async_tiles();
        __syncthreads();  // tile `it` is in LDS; every wave is done with the iteration before
        if (it + 1 < n_tiles) issue_tile(it + 1, (it + 1) & 1);
        const bool mine = it >= ta && it < tb;  // (the same for both waves of a block)
        const lds_char* stage = lds0 + (it & 1) * STAGE_BYTES;
        // LDS offsets are derived from these inside the iteration: kept across iterations they would
        // take more registers than the few vector instructions that compute them save
        int n_it = n, h_it = h;
        asm volatile("" : "+v"(n_it), "+v"(h_it));
        if (mine) {
            // rows = keys 8 * (r / 4) + 4 * h + r % 4 of the tile, column n = query row
            const lds_char* src = stage + role * TILE_BYTES;
            f32x16 acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const i32x4 a = *reinterpret_cast<const lds_i32x4*>(src + L::chunk_off(n_it, 2 * j + h_it));
                acc = Elem<E>::mma(a, res.c[j], acc);
            }
            // s * scale - LSE2 (what the exponential takes, chill_bwd_dq.py:314) or dP - delta
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = acc[r] * mult - sub;
            f32x4* out = reinterpret_cast<f32x4*>(xblock + role * X_BYTES);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++)
                out[r4 * 64 + lane] = f32x4{acc[4 * r4], acc[4 * r4 + 1], acc[4 * r4 + 2], acc[4 * r4 + 3]};
        }
        // the first operands of the accumulation do not depend on the exchange
        float a_k[2][DBW];
        auto read_operands = [&](int r, int buf) {
            const int rw = 8 * (r / 4) + 4 * h_it + (r % 4);
#pragma unroll
            for (int i = 0; i < DBW; i++)
                a_k[buf][i] = *reinterpret_cast<const lds_float*>(stage + L::elem_off(rw, 32 * (db0 + i) + n_it));
        };
        if (mine) read_operands(0, 0);
        __syncthreads();  // the products of this iteration are in LDS
        if (!mine) continue;

        f32x16 cs, cdp;
        {
            const f32x4* xs = reinterpret_cast<const f32x4*>(xblock);
            const f32x4* xd = reinterpret_cast<const f32x4*>(xblock + X_BYTES);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const f32x4 a = xs[r4 * 64 + lane], d = xd[r4 * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    cs[4 * r4 + i] = a[i];
                    cdp[4 * r4 + i] = d[i];
                }
            }
        }
        const bool full = (it >= fa) && (it < fb);
        const int k0 = (wg.start + it) * TK;
        // P = exp2(s * scale - LSE2), dS = P (dP - delta), dQ^T += K^T dS^T over this wave's head-dim
        // blocks; register by register, so that the vector work and the LDS reads of one register run
        // under the MFMAs of the one before
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float pv = fast_exp2(cs[r]);
            if (!full) {
                const int key = k0 + 8 * (r / 4) + 4 * h + (r % 4);
                const bool ok = (q_pos < seq_len) && (key < seq_len) && Mask<MASK>::pred(q_pos, key, seq_len, p.margs);
                pv = ok ? pv : 0.f;
            }
            const float ds = pv * cdp[r];
            if (r + 1 < 16) read_operands(r + 1, (r + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < DBW; i++) dq[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_k[r & 1][i], ds, dq[i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // lane (n, h) holds columns d = 32 * (db0 + i) + 8 * (r / 4) + 4 * h + r % 4 of ITS query row
    if (q_pos < p.T) {
        const bool valid = q_pos < seq_len;
        float* row = reinterpret_cast<float*>(dqbase + (int64_t)q_pos * p.sdq.t);
#pragma unroll
        for (int i = 0; i < DBW; i++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                f32x4 a;
#pragma unroll
                for (int e = 0; e < 4; e++) a[e] = valid ? dq[i][4 * g4 + e] * p.sm_scale : 0.f;
                *reinterpret_cast<f32x4*>(row + 32 * (db0 + i) + 8 * g4 + 4 * h) = a;
            }
    }
}

// ------------------------------------------------------------------------------------------ dK, dV
// One workgroup owns TKR = 32 * NW / 2 key rows; their K and V tiles sit in LDS for the whole
// kernel.  Streamed through the LDS ring: Q and dO tiles of 64 query rows with their LSE2 / delta,
// for every query head of the GQA group in turn (chill_bwd_dkdv.py:156).
//
// Waves work in pairs on one 32-key block: wave w takes the first 32 query rows of every streamed
// tile, wave w + NW/2 the second 32, each with its own dK^T / dV^T accumulators, which are summed
// through LDS at the end.  Splitting the QUERY axis inside a pair keeps the per-wave state (two
// 32 x D accumulators, no resident MFMA operands) within 256 registers, so two waves share a SIMD
// and one wave's vector work hides behind the other's MFMAs, with no redundant MFMA work.
// Four-wave workgroups are compiled for two per CU, those of head dims <= 64 (50 KiB of LDS) for three: 168 registers.
template <typename E, int D, int MASK, int NW, int NS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 4 ? (D <= 64 ? 3 : 2) : 1))) void dkdv_kernel(BwdParams p, int n_k_tiles, int total_items,
                                                       int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    typedef LdsTile<E, D> L;
    constexpr int NKB = NW / 2;      // 32-key blocks per workgroup
    constexpr int TKR = NKB * 32;    // resident key rows per workgroup
    constexpr int TQS = 64;          // streamed query rows per tile: 32 per wave of a pair
    constexpr int NT = NW * 64;
    constexpr int DB = (D + 31) / 32;
    constexpr int NJ = L::CH / 2;
    constexpr int KV_BYTES = L::bytes(TKR);
    constexpr int TILE_BYTES = L::bytes(TQS);
    constexpr int VEC_BYTES = TQS * 4;
    constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * VEC_BYTES;  // Q, dO, LSE2, delta
    constexpr int RING_OFF = 2 * KV_BYTES;                        // K, V tiles first
    static_assert(NS == 2, "two ring stages");
    // the pair exchange at the end reuses the LDS: 2 * NKB accumulators of DB * 16 * 64 floats (the tile
    // table allocates the larger of the two needs)
    extern __shared__ __attribute__((aligned(16))) char smem[];

    // (the 64-row workgroups of head dims up to 64 run three to a CU)
    const int item = xcd_contiguous_item(blockIdx.x, total_items, (NW == 4 && D <= 64) ? 3 : 1);
    if (item < 0) return;
    const int bh = item / n_k_tiles;
    // key tiles first-to-last: for causal-like masks the longest run first
    const int ktile = item % n_k_tiles;
    const int b = bh / p.H_kv;
    const int hkv = bh % p.H_kv;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kblk = wave % NKB;   // which 32-key block
    const int half = wave / NKB;   // which 32-row half of every streamed tile
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

    // resident K and V tiles
    {
        AsyncSwizzledLoader<E, D, TKR, NT> load_kv;
        const ET* kptr = reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h;
        const ET* vptr = reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;
        load_kv.init(p.sk.t, wave, lane);
        load_kv.issue(kptr + (int64_t)kb0 * p.sk.t, p.T - kb0, smem, wave, lane);
        load_kv.init(p.sv.t, wave, lane);
        load_kv.issue(vptr + (int64_t)kb0 * p.sv.t, p.T - kb0, smem + KV_BYTES, wave, lane);
    }

    AsyncSwizzledLoader<E, D, TQS, NT> load_q, load_do;
    load_q.init(p.sq.t, wave, lane);
    load_do.init(p.sdo.t, wave, lane);
    // Iterations run over (group head g, q-tile).  The tile to issue next is tracked incrementally —
    // pointers advance by one tile, and are rebuilt only when the next query head starts — so that
    // issuing costs a handful of scalar instructions per iteration.
    struct {
        const ET* q;
        const ET* d_o;
        const float* lse;
        const float* del;
        int rows_left;  // rows from the tile's first row to the end of the tensor
        int tile;       // index inside [0, n_tiles)
        int g;
    } nxt;
    auto start_head = [&](int g) {
        const int hq = hkv * p.group + g;
        const int q0 = wg.start * TQS;
        nxt.q = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hq * p.sq.h + (int64_t)q0 * p.sq.t;
        nxt.d_o = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hq * p.sdo.h + (int64_t)q0 * p.sdo.t;
        nxt.lse = p.lse + b * p.lse_b + hq * p.lse_h + q0;
        nxt.del = p.delta + b * p.delta_b + hq * p.delta_h + q0;
        nxt.rows_left = p.T - q0;
        nxt.tile = 0;
        nxt.g = g;
    };
    int n_issued = 0;
    // move to the tile after the one just issued; past the end the last tile stays selected
    auto advance = [&]() {
        n_issued++;
        if (n_issued >= n_iters) return;
        if (nxt.tile + 1 == n_tiles) {
            start_head(nxt.g + 1);
        } else {
            nxt.q += TQS * p.sq.t;
            nxt.d_o += TQS * p.sdo.t;
            nxt.lse += TQS;
            nxt.del += TQS;
            nxt.rows_left -= TQS;
            nxt.tile++;
        }
    };
    auto issue_next = [&](int st_index) {
        char* st = smem + RING_OFF + st_index * STAGE_BYTES;
        load_q.issue(nxt.q, nxt.rows_left, st, wave, lane);
        load_do.issue(nxt.d_o, nxt.rows_left, st + TILE_BYTES, wave, lane);
        if (wave == NW - 1) {
            // LSE2 and delta of the tile's rows; rows past the end of the tensor read as zero
            char* vec = st + 2 * TILE_BYTES;
            if (lane < nxt.rows_left) {
                async_load4(nxt.lse, lane * 4, lds_address(vec));
                async_load4(nxt.del, lane * 4, lds_address(vec + VEC_BYTES));
            } else {
                reinterpret_cast<float*>(vec)[lane] = 0.f;
                reinterpret_cast<float*>(vec + VEC_BYTES)[lane] = 0.f;
            }
        }
        advance();
    };
    start_head(0);
    if (n_iters > 0) issue_next(0);

    const int kw = kb0 + 32 * kblk;
    const int k_pos = kw + n;
    const Range vis = visible_range<MASK, false>(k_pos, seq_len, p.margs);  // the queries that see this lane's key
    OperandOffsets<E, D> ofs;
    ofs.init(lane);

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    if (kw < seq_len) wr = tile_range<MASK, false>(kw, 32, TQS, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            dk[i][r] = 0.f;
            dv[i][r] = 0.f;
        }
    const float scale = p.scale_log2;
    const float masked_score = scale < 0.f ? INFINITY : -INFINITY;  // times the scale: -inf
    const lds_char* lds0 = (const lds_char*)smem;
    const lds_char* k_tile = lds0;
    const lds_char* v_tile = lds0 + KV_BYTES;

    // Operand addresses.  Where a tile's 32-row blocks are affine, everything wave-dependent (the key
    // block, the half of the streamed tile, the ring's place behind K and V) goes into per-lane pointers
    // once, and the loop is unrolled over the two ring stages: every LDS read of the loop then is a
    // loop-invariant register plus a constant in the instruction's offset field.
    // Not for the 4-wave workgroups of head dims <= 64: they run three to a CU at <= 168 registers, which the
    // pointers would exceed (B4 H32 T8192 D64 causal: 2.29 ms as they are, 2.38 folded and chained, 2.46 folded only)
    constexpr bool kFold = L::kBlockAffine && Elem<E>::k16 && (NW == 8 || D >= 128);
    // operands read ahead in a block's MFMA chain (folded path only).  C3: 4.05 ms in the compiler's order,
    // 3.97 with the S / dP part of the chain two ahead, 3.90 with the whole chain two ahead; three ahead
    // 3.98, the transposed operands three or four ahead 4.10 / 4.17 (more requests in flight per wave
    // only lengthen the queue of the LDS, which is busy 45 % of the time)
    constexpr int kPrefetch = 2 < NJ ? 2 : NJ;
    constexpr int kPrefetchTr = kPrefetch;
    static_assert(kPrefetchTr >= kPrefetch && kPrefetch >= 1, "read-ahead distances");
    OperandPointers<E, D> at_k, at_q;  // K / V rows of this wave's key block; Q / dO rows of its half
    const lds_char* vec0 = lds0 + RING_OFF + 2 * TILE_BYTES + (32 * half + 4 * h) * 4;  // LSE2 / delta of the lane's 16 rows
    if constexpr (kFold) {
        at_k.template init<false>(ofs, lds0 + kblk * L::BLOCK_BYTES);
        at_q.template init<true>(ofs, lds0 + RING_OFF + half * L::BLOCK_BYTES);
        asm volatile("" : "+v"(vec0));
    }

    int tile = -1;  // position of iteration `it` inside the q-tile range (it % n_tiles)
    // iteration `it` consumes ring stage ST = it % 2
    auto iteration = [&](auto st_tag, int it) {
        constexpr int ST = decltype(st_tag)::value;
        wait_async_tiles();
        __syncthreads();
        tile = tile + 1 == n_tiles ? 0 : tile + 1;
        const bool in_block = !(tile < ta || tile >= tb);
        // the two waves that share a SIMD issue their loads at different points of the iteration, so
        // that one of them keeps the matrix pipe busy while the other sits in the memory pipeline
        const bool issue_late = in_block && half == 1;
        if (!issue_late) {
            if (it + 1 < n_iters) issue_next(1 - ST);
        }
        if (!in_block) return;
        const lds_char* q_tile = lds0 + RING_OFF + ST * STAGE_BYTES;
        const lds_char* do_tile = q_tile + TILE_BYTES;
        const lds_char* vec = vec0 + ST * STAGE_BYTES;
        constexpr int Q_AT = ST * STAGE_BYTES, DO_AT = Q_AT + TILE_BYTES;
        const bool full = (tile >= fa) && (tile < fb);
        const int q0 = (wg.start + tile) * TQS + 32 * half;

        // One 32 x 32 block.  The vector work is split in two parts, each written next to a GEMM that
        // does not depend on it: P = exp2(S * scale - LSE2) after dP = dO V^T has been issued,
        // dS = P (dP - delta) after dV^T += dO^T P.  All MFMA operands come from LDS.
        // Masked entries get a score of -inf (times the sign of the scale) in a branch of their own, so
        // that the rest of the block is the same straight-line code for full and partial tiles.
        f32x4 lse4[4], del4[4];
        auto read_lse = [&]() {
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++)
                lse4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + 32 * g4);
        };
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            s[r] = 0.f;
            dp[r] = 0.f;
        }
        auto mask_scores = [&]() {
            if constexpr (Mask<MASK>::kRowIsRange) {
                fill_outside_range(s, vis.lo, vis.hi, q0 + 4 * h, masked_score);
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int q = q0 + 8 * (r / 4) + 4 * h + (r % 4);
                    const bool ok = (q < seq_len) && (k_pos < seq_len) && Mask<MASK>::pred(q, k_pos, seq_len, p.margs);
                    s[r] = ok ? s[r] : masked_score;
                }
            }
            // a row that attends to nothing has LSE2 = -inf and only masked entries
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float l = lse4[r / 4][r % 4];
                lse4[r / 4][r % 4] = (l == -INFINITY) ? 0.f : l;
            }
        };
        if constexpr (kFold) {
            // The block's 2 NJ + 4 DB MFMAs — S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS — as one
            // chain whose LDS operands are read kPrefetch steps ahead, in this order and no other: left to
            // itself the compiler reads most operands right before their MFMA, and the wave waits out the
            // LDS latency again and again.  The vector work rides along: the exponentials on the dP
            // steps, dS on the dV^T steps.
            constexpr int N1 = NJ, N2 = 2 * NJ, N3 = N2 + 2 * DB, N4 = N3 + 2 * DB;
            i32x4 opa[N4], opb[N2];
            auto fetch = [&](auto t_tag) {
                constexpr int t = decltype(t_tag)::value;
                if constexpr (t < N1) {
                    opa[t] = at_q.row_chunk(Q_AT, t);
                    opb[t] = at_k.row_chunk(0, t);
                } else if constexpr (t < N2) {
                    opa[t] = at_q.row_chunk(DO_AT, t - N1);
                    opb[t] = at_k.row_chunk(KV_BYTES, t - N1);
                } else if constexpr (t < N3) {
                    opa[t] = at_q.tr_operand(DO_AT, (t - N2) / DB, (t - N2) % DB);
                } else if constexpr (t < N4) {
                    opa[t] = at_q.tr_operand(Q_AT, (t - N3) / DB, (t - N3) % DB);
                }
            };
            // operand i is read at step i - kPrefetch (row-wise pairs, 8 registers) or i - kPrefetchTr
            // (transposed operands, 4 registers); what falls before step 0 is read up front
            auto ahead = [&](auto t_tag) {
                constexpr int t = decltype(t_tag)::value;
                if constexpr (t + kPrefetch < N2) fetch(std::integral_constant<int, t + kPrefetch>{});
                if constexpr (t + kPrefetchTr >= N2) fetch(std::integral_constant<int, t + kPrefetchTr>{});
            };
            static_for<kPrefetch>([&](auto t) { fetch(t); });
            __builtin_amdgcn_sched_barrier(0);
            static_for<NJ>([&](auto t) {
                s = Elem<E>::mma(opa[t], opb[t], s);
                asm volatile("" : "+v"(s));  // keeps the MFMA at this place of the chain
                ahead(t);
                if constexpr (t == NJ / 2) read_lse();  // needed from the first step of the dP part on
                __builtin_amdgcn_sched_barrier(0);
            });
            if (!full) mask_scores();
            constexpr int PER = (16 + NJ - 1) / NJ;  // exponentials per dP step
            i32x4 pb[2], dsb[2];
            static_for<NJ>([&](auto t) {
                dp = Elem<E>::mma(opa[N1 + t], opb[N1 + t], dp);
                asm volatile("" : "+v"(dp));
                ahead(std::integral_constant<int, N1 + t>{});
#pragma unroll
                for (int r = PER * t; r < PER * (t + 1) && r < 16; r++)
                    s[r] = fast_exp2(__builtin_fmaf(s[r], scale, -lse4[r / 4][r % 4]));
                if constexpr (t == NJ / 2) {
#pragma unroll
                    for (int g4 = 0; g4 < 4; g4++)
                        del4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + VEC_BYTES + 32 * g4);
                }
                if constexpr (t == NJ - 1) pack_block<E>(s, pb);
                __builtin_amdgcn_sched_barrier(0);
            });
            constexpr int PERD = (16 + 2 * DB - 1) / (2 * DB);  // entries of dS per dV^T step
            static_for<2 * DB>([&](auto u) {
                constexpr int db = u % DB;
                dv[db] = Elem<E>::mma(opa[N2 + u], pb[u / DB], dv[db]);
                asm volatile("" : "+v"(dv[db]));
                ahead(std::integral_constant<int, N2 + u>{});
#pragma unroll
                for (int r = PERD * u; r < PERD * (u + 1) && r < 16; r++) dp[r] = s[r] * (dp[r] - del4[r / 4][r % 4]);
                if constexpr (u == 2 * DB - 1) pack_block<E>(dp, dsb);
                __builtin_amdgcn_sched_barrier(0);
            });
            if (issue_late) {
                if (it + 1 < n_iters) issue_next(1 - ST);
            }
            static_for<2 * DB>([&](auto u) {
                constexpr int db = u % DB;
                dk[db] = Elem<E>::mma(opa[N3 + u], dsb[u / DB], dk[db]);
                asm volatile("" : "+v"(dk[db]));
                ahead(std::integral_constant<int, N3 + u>{});
                __builtin_amdgcn_sched_barrier(0);
            });
        } else {
            read_lse();
#pragma unroll
            for (int j = 0; j < NJ; j++)
                s = Elem<E>::mma(ofs.row_chunk(q_tile, half, j, lane), ofs.row_chunk(k_tile, kblk, j, lane), s);
            if (!full) mask_scores();
#pragma unroll
            for (int j = 0; j < NJ; j++)
                dp = Elem<E>::mma(ofs.row_chunk(do_tile, half, j, lane), ofs.row_chunk(v_tile, kblk, j, lane), dp);
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = fast_exp2(__builtin_fmaf(s[r], scale, -lse4[r / 4][r % 4]));
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++)
                del4[g4] = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + VEC_BYTES + 32 * g4);
            mma_transposed<E, D>(do_tile, half, ofs, s, dv, lane);  // dV^T += dO^T P
            if (issue_late) {
                if (it + 1 < n_iters) issue_next(1 - ST);
            }
#pragma unroll
            for (int r = 0; r < 16; r++) dp[r] = s[r] * (dp[r] - del4[r / 4][r % 4]);
            mma_transposed<E, D>(q_tile, half, ofs, dp, dk, lane);  // dK^T += Q^T dS
        }
    };
    for (int it = 0; it < n_iters; it += 2) {
        iteration(std::integral_constant<int, 0>{}, it);
        if (it + 1 < n_iters) iteration(std::integral_constant<int, 1>{}, it + 1);
    }

    // Sum the two waves of a pair through LDS and store: the waves of the second half hand their dK^T
    // partials to the first half and receive its dV^T partials, so that every wave finishes one 32 x D
    // block.  The block then goes through LDS once more, row-major at a padded pitch, so that a store
    // instruction writes whole rows (16 lanes x 16 bytes per 256-byte row) instead of 8 bytes of 32 rows.
    wait_async_tiles();
    constexpr int XCH_FLOATS = DB * 16 * 64;  // one wave's accumulator
    float* xch_k = reinterpret_cast<float*>(smem) + kblk * XCH_FLOATS;
    float* xch_v = reinterpret_cast<float*>(smem) + (NKB + kblk) * XCH_FLOATS;
    f32x16(&give)[DB] = half == 1 ? dk : dv;
    f32x16(&keep)[DB] = half == 1 ? dv : dk;
    float* give_to = (half == 1 ? xch_k : xch_v) + lane;
    float* take_from = (half == 1 ? xch_v : xch_k) + lane;
    __syncthreads();  // everyone is done with the tiles
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) give_to[(db * 16 + r) * 64] = give[db][r];
    __syncthreads();
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) keep[db][r] += take_from[(db * 16 + r) * 64];

    ET* out = half == 1 ? dvbase : dkbase;
    const int64_t out_stride = half == 1 ? p.sdv.t : p.sdk.t;
    const float mult = half == 1 ? 1.f : p.sm_scale;
    const bool valid = k_pos < seq_len;
    if constexpr (!Elem<E>::k16) {
        if (k_pos < p.T) store_row_transposed<E, D>(out + (int64_t)k_pos * out_stride, keep, mult, valid, h);
    } else {
        // the region this wave just read is its own from here on: stage the finished block there
        constexpr int RB = D * 2;       // bytes per row
        constexpr int PITCH = RB + 8;   // 8-byte writes of 32 consecutive rows spread over all banks
        constexpr int CH = RB / 16;     // 16-byte chunks per row
        static_assert(32 * PITCH <= XCH_FLOATS * 4, "the staged block fits the wave's exchange region");
        char* stage = reinterpret_cast<char*>(half == 1 ? xch_v : xch_k);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = 32 * db + 8 * g + 4 * h;
                if (D >= 32 || d0 < D) {
                    f32x4 vals;
#pragma unroll
                    for (int e = 0; e < 4; e++) vals[e] = valid ? keep[db][4 * g + e] * mult : 0.f;
                    *reinterpret_cast<i32x2*>(stage + n * PITCH + d0 * 2) = Elem<E>::pack4(vals);
                }
            }
        constexpr int ROWS_PER_STEP = 64 / CH;  // 4 (D = 128) .. 32 (D = 16)
        // (what is derived from the lane index here is derived again, not kept from the prologue through
        // the whole loop: at 256 registers that cost a slot in scratch memory)
        int lane_e = threadIdx.x & 63;
        asm volatile("" : "+v"(lane_e));
#pragma unroll
        for (int row0 = 0; row0 < 32; row0 += ROWS_PER_STEP) {
            const int row = row0 + lane_e / CH, c = lane_e % CH;
            // PITCH is a multiple of 8 only: two 8-byte reads
            const i32x2 lo = *reinterpret_cast<const i32x2*>(stage + row * PITCH + c * 16);
            const i32x2 hi = *reinterpret_cast<const i32x2*>(stage + row * PITCH + c * 16 + 8);
            if (kw + row < p.T)
                *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(out + (int64_t)(kw + row) * out_stride) + c * 16) =
                    i32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    }
}

// ------------------------------------------------------------------------------------------ dK, dV (wide rows)
// Variant for rows too long for the paired kernel's LDS budget (more than 256 bytes per row: fp32 at
// head dims 128 and 256).  A 32-key block keeps 32 x D of K, 32 x D of V and two 32 x D accumulators:
// four times D registers per lane in one wave, more than a wave has from D = 128 on.  So SPLIT waves
// share a block and each holds a quarter of that state per pair of waves:
//   * wave g of the block computes a PARTIAL product over its share of the head dim, S = Q K^T for
//     even g and dP = dO V^T for odd g, from its resident slice of K or V (B operands);
//   * the partial products meet in LDS; behind a barrier every wave of the block adds them up and
//     computes P and dS for itself (vector work that is small next to fp32 MFMAs);
//   * wave g accumulates the head-dim blocks [g * DB / SPLIT, (g + 1) * DB / SPLIT) of dV^T += dO^T P
//     and dK^T += Q^T dS.
// Every wave issues the same number of MFMAs and none is issued twice.  Streamed through the LDS ring:
// Q and dO tiles of 32 query rows, for every query head of the GQA group in turn
// (chill_bwd_dkdv.py:156), with the LSE2 / delta of those rows.
template <typename E, int D, int MASK, int NW, int SPLIT, int NS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(D >= 256 ? 1 : 2))) void dkdv_split_kernel(BwdParams p, int n_k_tiles, int total_items,
                                                        int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    typedef LdsTile<E, D> L;
    static_assert(!Elem<E>::k16, "fp32 rows (16-bit rows of this length have a kernel of their own)");
    constexpr int TQS = 32;
    constexpr int NKB = NW / SPLIT;   // 32-key blocks per workgroup
    constexpr int TKR = NKB * 32;     // key rows per workgroup
    constexpr int NT = NW * 64;
    constexpr int DB = D / 32;
    constexpr int DBW = DB / SPLIT;   // head-dim blocks a wave accumulates
    constexpr int PARTS = SPLIT / 2;  // slices of the head dim in the partial products
    constexpr int NJW = (L::CH / 2) / PARTS;  // 16-byte chunk pairs of a slice
    constexpr int TILE_BYTES = L::bytes(TQS);
    constexpr int VEC_BYTES = TQS * 4;
    constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * VEC_BYTES;  // Q, dO, LSE2, delta
    constexpr int X_BYTES = 16 * 64 * 4;                         // one partial product
    static_assert(NS == 2, "two ring stages");
    static_assert(SPLIT % 2 == 0 && DB % SPLIT == 0 && NW % SPLIT == 0, "whole shares");
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
    const int kblk = wave % NKB;
    const int g = wave / NKB;       // place among the waves of the block
    const int role = g & 1;         // 0: S from K, 1: dP from V
    const int part = g >> 1;        // slice of the head dim in the partial product
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
    // iteration it = (group head, q-tile): stage it % 2
    auto issue_iter = [&](int it, int st_index) {
        const int gh = it / n_tiles;
        const int q0 = (wg.start + it % n_tiles) * TQS;
        const int hq = hkv * p.group + gh;
        char* st = smem + st_index * STAGE_BYTES;
        const ET* qptr = reinterpret_cast<const ET*>(p.q) + b * p.sq.b + hq * p.sq.h;
        const ET* doptr = reinterpret_cast<const ET*>(p.d_o) + b * p.sdo.b + hq * p.sdo.h;
        load_q.issue(qptr + (int64_t)q0 * p.sq.t, p.T - q0, st, wave, lane);
        load_do.issue(doptr + (int64_t)q0 * p.sdo.t, p.T - q0, st + TILE_BYTES, wave, lane);
        if (wave == 0) {
            // LSE2 and delta of the tile's rows; rows past the end of the tensor read as zero
            const float* lse = p.lse + b * p.lse_b + hq * p.lse_h + q0;
            const float* del = p.delta + b * p.delta_b + hq * p.delta_h + q0;
            char* vec = st + 2 * TILE_BYTES;
            if (lane < TQS) {
                if (q0 + lane < p.T) {
                    async_load4(lse, lane * 4, lds_address(vec));
                    async_load4(del, lane * 4, lds_address(vec + VEC_BYTES));
                } else {
                    reinterpret_cast<float*>(vec)[lane] = 0.f;
                    reinterpret_cast<float*>(vec + VEC_BYTES)[lane] = 0.f;
                }
            }
        }
    };
    if (n_iters > 0) issue_iter(0, 0);

    // this wave's slice of K (role 0) or V (role 1): chunk pairs [part * NJW, (part + 1) * NJW) of the
    // block's 32 rows as B operands; rows past the end of the tensor read as zero
    const int kw = kb0 + 32 * kblk;
    const int k_pos = kw + n;
    i32x4 res[NJW];
    {
        const ET* src = role == 0 ? reinterpret_cast<const ET*>(p.k) + b * p.sk.b + hkv * p.sk.h
                                  : reinterpret_cast<const ET*>(p.v) + b * p.sv.b + hkv * p.sv.h;
        const int64_t stride = role == 0 ? p.sk.t : p.sv.t;
#pragma unroll
        for (int j = 0; j < NJW; j++) {
            i32x4 val = {0, 0, 0, 0};
            if (k_pos < p.T)
                val = *reinterpret_cast<const i32x4*>(reinterpret_cast<const char*>(src + (int64_t)k_pos * stride) +
                                                      (2 * (part * NJW + j) + h) * 16);
            res[j] = val;
        }
    }

    TileRange wr = {wg.start, wg.start, wg.start, wg.start};
    if (kw < seq_len) wr = tile_range<MASK, false>(kw, 32, TQS, seq_len, wave_has_full_blocks != 0, p.margs);
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    f32x16 dk[DBW], dv[DBW];
#pragma unroll
    for (int i = 0; i < DBW; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            dk[i][r] = 0.f;
            dv[i][r] = 0.f;
        }
    const float scale = p.scale_log2;
    const lds_char* lds0 = (const lds_char*)smem;
    // the partial products of block kblk: SPLIT slots of 16 x 64 floats, register r of lane l at
    // ((r / 4) * 64 + l) * 16 + (r % 4) * 4
    char* xblock = smem + 2 * STAGE_BYTES + kblk * SPLIT * X_BYTES;
    // this wave's head-dim blocks in the accumulation: columns 32 * (g * DBW + i) + n of the Q / dO tiles
    const int db0 = g * DBW;

    int tile = -1;  // position of iteration `it` inside the q-tile range (it % n_tiles)
    for (int it = 0; it < n_iters; it++) {
        wait_async_tiles();
        __syncthreads();  // tile `it` is in LDS; every wave is done with the iteration before
        tile = tile + 1 == n_tiles ? 0 : tile + 1;
        const bool mine = tile >= ta && tile < tb;  // (the same for all waves of a block)
        const lds_char* stage = lds0 + (it & 1) * STAGE_BYTES;
        const int q0 = (wg.start + tile) * TQS;
        // The wave that produces S (dP) also subtracts the LSE2 (delta) of its query rows, rows
        // 8 * (r / 4) + 4 * h + r % 4 of the tile: every wave reads one of the two vectors and only where
        // it produces.
        if (it + 1 < n_iters) issue_iter(it + 1, (it + 1) & 1);
        // LDS offsets are derived from these inside the iteration: kept across iterations they would
        // take more registers than the few vector instructions that compute them save
        int n_it = n, h_it = h;
        asm volatile("" : "+v"(n_it), "+v"(h_it));
        if (mine) {
            const lds_char* src = stage + role * TILE_BYTES;
            f32x16 part_acc;
#pragma unroll
            for (int r = 0; r < 16; r++) part_acc[r] = 0.f;
#pragma unroll
            for (int j = 0; j < NJW; j++) {
                const i32x4 a = *reinterpret_cast<const lds_i32x4*>(src + L::chunk_off(n_it, 2 * (part * NJW + j) + h_it));
                part_acc = Elem<E>::mma(a, res[j], part_acc);
            }
            float vec16[16];
            const lds_float* vec = reinterpret_cast<const lds_float*>(stage + 2 * TILE_BYTES) + role * TQS;
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const f32x4 v4 = *reinterpret_cast<const __attribute__((address_space(3))) f32x4*>(vec + 8 * g4 + 4 * h_it);
#pragma unroll
                for (int e = 0; e < 4; e++) vec16[4 * g4 + e] = v4[e];
            }
            // s * scale - LSE2 (what the exponential takes, chill_bwd_dkdv.py:378) or dP - delta
            const float mult = role == 0 ? scale : 1.f;
            const bool sub = part == 0;
#pragma unroll
            for (int r = 0; r < 16; r++) part_acc[r] = part_acc[r] * mult - (sub ? vec16[r] : 0.f);
            f32x4* out = reinterpret_cast<f32x4*>(xblock + g * X_BYTES);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++)
                out[r4 * 64 + lane] = f32x4{part_acc[4 * r4], part_acc[4 * r4 + 1], part_acc[4 * r4 + 2], part_acc[4 * r4 + 3]};
        }
        // the first operands of the accumulation do not depend on the exchange
        float a_do[2][DBW], a_q[2][DBW];
        auto read_operands = [&](int r, int buf) {
            const int rw = 8 * (r / 4) + 4 * h_it + (r % 4);
#pragma unroll
            for (int i = 0; i < DBW; i++) {
                const int off = L::elem_off(rw, 32 * (db0 + i) + n_it);
                a_do[buf][i] = *reinterpret_cast<const lds_float*>(stage + TILE_BYTES + off);
                a_q[buf][i] = *reinterpret_cast<const lds_float*>(stage + off);
            }
        };
        if (mine) read_operands(0, 0);
        __syncthreads();  // the partial products of this iteration are in LDS
        if (!mine) continue;

        f32x16 cs, cdp;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            cs[r] = 0.f;
            cdp[r] = 0.f;
        }
#pragma unroll
        for (int e = 0; e < PARTS; e++) {
            const f32x4* xs = reinterpret_cast<const f32x4*>(xblock + (2 * e) * X_BYTES);
            const f32x4* xd = reinterpret_cast<const f32x4*>(xblock + (2 * e + 1) * X_BYTES);
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const f32x4 a = xs[r4 * 64 + lane], d = xd[r4 * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    cs[4 * r4 + i] += a[i];
                    cdp[4 * r4 + i] += d[i];
                }
            }
        }
        const bool full = (tile >= fa) && (tile < fb);
        // P = exp2(s * scale - LSE2) and dS = P (dP - delta) (the sums hold the arguments), then
        // dV^T += dO^T P and dK^T += Q^T dS over this wave's head-dim blocks: the contraction runs over the
        // 32 query rows, two per MFMA (rows 8 * (r / 4) + r % 4 and that + 4).  Register by register, so
        // that the vector work and the LDS reads of one register run under the MFMAs of the one before.
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float pv = fast_exp2(cs[r]);
            if (!full) {
                const int qq = q0 + 8 * (r / 4) + 4 * h + (r % 4);
                const bool ok = (qq < seq_len) && (k_pos < seq_len) && Mask<MASK>::pred(qq, k_pos, seq_len, p.margs);
                pv = ok ? pv : 0.f;
            }
            const float ds = pv * cdp[r];
            if (r + 1 < 16) read_operands(r + 1, (r + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < DBW; i++) {
                dv[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_do[r & 1][i], pv, dv[i], 0, 0, 0);
                dk[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_q[r & 1][i], ds, dk[i], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // lane (n, h) holds columns d = 32 * (db0 + i) + 8 * (r / 4) + 4 * h + r % 4 of ITS key row
    if (k_pos < p.T) {
        const bool valid = k_pos < seq_len;
        float* dkrow = reinterpret_cast<float*>(dkbase + (int64_t)k_pos * p.sdk.t);
        float* dvrow = reinterpret_cast<float*>(dvbase + (int64_t)k_pos * p.sdv.t);
#pragma unroll
        for (int i = 0; i < DBW; i++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const int d0 = 32 * (db0 + i) + 8 * g4 + 4 * h;
                f32x4 a, c;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    a[e] = valid ? dk[i][4 * g4 + e] * p.sm_scale : 0.f;
                    c[e] = valid ? dv[i][4 * g4 + e] : 0.f;
                }
                *reinterpret_cast<f32x4*>(dkrow + d0) = a;
                *reinterpret_cast<f32x4*>(dvrow + d0) = c;
            }
    }
}

// One (mask, tile shape): SMALL selects the table row for grids that would not fill the chip, REGS the one of
// dkdv_regs_kernel where the shape has both kernels.
template <typename E, int D, int MASK_ID, bool SMALL, bool REGS = false>
int launch_dkdv_shape(const BwdParams& p, hipStream_t stream) {
    constexpr TileConfig cfg = dkdv_tile_config(MASK_ID, D, Elem<E>::kDType, SMALL, REGS);
    constexpr int CB = (REGS && dkdv_regs_is_optional(D, Elem<E>::kDType)) ? kDkdvRegsBlocks128 : dkdv_regs_blocks(D, Elem<E>::kDType);
    constexpr bool paired = dkdv_is_paired(D, Elem<E>::kDType) && CB == 0;
    static_assert(CB > 0 ? (cfg.rows == 128 * CB && cfg.streamed == 32 && cfg.waves == 4)
                         : paired ? (cfg.rows * 2 == cfg.waves * 32 && cfg.streamed == 64)
                                  : (cfg.rows * dkdv_split(D) == cfg.waves * 32 && cfg.streamed == 32),
                  "tile table and kernel shape disagree");
    const int n_k_tiles = cdiv(p.T, cfg.rows);
    const int64_t total64 = (int64_t)p.B * p.H_kv * n_k_tiles;
    if (total64 > ((int64_t)1 << 30)) return CHILL_ERR_TOO_LARGE;
    const int total = (int)total64;
    dim3 grid(cdiv(total, 8) * 8), block(cfg.waves * 64);
    static_assert(!paired || cfg.lds_bytes >= dkdv_paired_exchange_bytes(D) * cfg.waves / 8, "LDS for the pair exchange");
    void (*kern)(BwdParams, int, int, int);
    if constexpr (CB > 0)
        kern = dkdv_regs_kernel<E, D, MASK_ID, CB, dkdv_regs_stages(D)>;
    else if constexpr (paired)
        kern = dkdv_kernel<E, D, MASK_ID, cfg.waves, 2>;
    else
        kern = dkdv_split_kernel<E, D, MASK_ID, cfg.waves, dkdv_split(D), 2>;
    // mask rule order is (q tile, k tile): the streamed tile is the q tile here
    const bool hfb = Mask<MASK_ID>::has_full_blocks(cfg.streamed, CB > 0 ? 32 * CB : 32, p.T, p.margs);
    if (cfg.lds_bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                cfg.lds_bytes) != hipSuccess)
            return CHILL_ERR_HIP;
    }
    hipLaunchKernelGGL(kern, grid, block, cfg.lds_bytes, stream, p, n_k_tiles, total, hfb ? 1 : 0);
    return (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
}

template <typename E, int D>
int launch_dkdv(const BwdParams& p, int mask_id, hipStream_t stream) {
    int64_t max_stride = p.sq.t > p.sdo.t ? p.sq.t : p.sdo.t;
    if (p.sk.t > max_stride) max_stride = p.sk.t;
    if (p.sv.t > max_stride) max_stride = p.sv.t;
    if (max_stride * Elem<E>::kBytes * 256 >= ((int64_t)1 << 31)) return CHILL_ERR_TOO_LARGE;
    int status = CHILL_ERR_BAD_MASK;
    CHILL_DISPATCH_MASK(mask_id, {
        // the table has a row of its own for small grids where that row differs
        constexpr bool has_small_row = dkdv_tile_config(MASK_ID, D, Elem<E>::kDType, true).waves !=
                                       dkdv_tile_config(MASK_ID, D, Elem<E>::kDType, false).waves;
        bool small = false;
        constexpr bool served = bwd_small_serves(D, Elem<E>::kDType, CHILL_PASS_DKDV);
        if constexpr (served) small = bwd_takes_small(MASK_ID, (long long)p.B * p.H_kv, p.T, D, Elem<E>::kDType, CHILL_PASS_DKDV);
        bool regs = false;
        if constexpr (dkdv_regs_is_optional(D, Elem<E>::kDType))
            regs = dkdv_takes_regs(MASK_ID, p.margs.a0, mask_band_keys(MASK_ID, p.margs.a0, p.margs.a1), D, (long long)p.B * p.H_kv, p.T);
        if (small) {
            if constexpr (served) status = launch_bwd_small<E, D, MASK_ID, 2>(p, stream);
        } else if (regs) {
            if constexpr (dkdv_regs_is_optional(D, Elem<E>::kDType)) status = launch_dkdv_shape<E, D, MASK_ID, false, true>(p, stream);
        } else if constexpr (has_small_row) {
            status = dkdv_takes_small_row((long long)p.B * p.H_kv, p.T) ? launch_dkdv_shape<E, D, MASK_ID, true>(p, stream)
                                                                        : launch_dkdv_shape<E, D, MASK_ID, false>(p, stream);
        } else {
            status = launch_dkdv_shape<E, D, MASK_ID, false>(p, stream);
        }
    });
    return status;
}

}  // namespace chill
