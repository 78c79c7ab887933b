// Forward kernel: O = softmax(mask(Q K^T * scale)) V and LSE2, one workgroup per (batch, head,
// q-tile) — the gfx950 counterpart of the reference's Triton program _chill_attn_fwd
// (chill_attention/chill_fwd.py:21-359).
//
// Each wave owns 32 query rows.  It keeps Q^T as MFMA B operands in registers and computes the
// TRANSPOSED score block S^T = K Q^T, so that in the accumulator layout one lane holds scores of
// a single query row: the running max / sum of the online softmax (chill_fwd.py:214-226) are
// per-lane scalars, and the only cross-lane step is one v_permlane32_swap per tile.  P^T in
// accumulator layout is directly the B operand of O^T += V^T P^T; V^T comes out of LDS through
// the transposing read (ds_read_b64_tr_b16), so V is staged exactly like K.
//
// K/V tiles are staged through double-buffered, XOR-swizzled LDS by the whole workgroup; the
// global loads of tile i+1 are in flight while tile i is consumed.
//
// Tile skipping and the predicate-free path follow chill_fwd.py:131-139 and :161-185, evaluated
// per WAVE (32 rows): a wave skips streamed tiles outside its own k-range and drops the predicate
// inside its own full range.  The workgroup stages the hull of its waves' ranges.
#pragma once

#include "chill_device.h"
#include "chill_params.h"
#include "chill_tiles.h"

namespace chill {

template <typename E, int D, int MASK, int NW, int TK>
__global__ __launch_bounds__(NW * 64) void fwd_kernel(FwdParams p, int n_q_tiles, int total_items,
                                                      int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    using M = Mask<MASK>;
    constexpr int TQ = NW * 32;
    constexpr int NT = NW * 64;
    constexpr int KB = TK / 32;         // 32-key blocks per streamed tile
    constexpr int DB = (D + 31) / 32;   // 32-wide blocks of the head dim
    constexpr int TILE_BYTES = LdsTile<E, D>::bytes(TK);
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int item = xcd_contiguous_item(blockIdx.x, total_items);
    if (item < 0) return;
    const int bh = item / n_q_tiles;
    // q-tiles of one head are issued last-first: for causal-like masks the longest run first
    const int qt = n_q_tiles - 1 - item % n_q_tiles;
    const int b = bh / p.H;
    const int hd = bh % p.H;
    const int hkv = hd / p.group;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
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

    const int qw = qb + 32 * wave;
    Resident<E, D> qf;
    load_resident<E, D>(qf, qptr + (int64_t)qw * p.sq.t, p.sq.t, p.T - qw, lane);

    const TileRange wg = tile_range<MASK, true>(qb, TQ, TK, seq_len, false, p.margs);
    TileRange wr = {0, 0, 0, 0};
    if (qw < seq_len) wr = tile_range<MASK, true>(qw, 32, TK, seq_len, wave_has_full_blocks != 0, p.margs);

    f32x16 o[DB];
#pragma unroll
    for (int i = 0; i < DB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] = 0.f;
    float m_run = -INFINITY;
    float l_run = 0.f;
    const int q_pos = qw + n;
    const float scale = p.scale_log2;

    TileStager<E, D, TK, NT> stage_k, stage_v;
    {
        int k0 = wg.start * TK;
        stage_k.fetch(kptr + (int64_t)k0 * p.sk.t, p.sk.t, p.T - k0, tid);
        stage_v.fetch(vptr + (int64_t)k0 * p.sv.t, p.sv.t, p.T - k0, tid);
    }

    for (int kt = wg.start; kt < wg.end; kt++) {
        char* lds_k = smem + ((kt - wg.start) & 1) * 2 * TILE_BYTES;
        char* lds_v = lds_k + TILE_BYTES;
        stage_k.commit(lds_k, tid);
        stage_v.commit(lds_v, tid);
        __syncthreads();
        if (kt + 1 < wg.end) {
            int k1 = (kt + 1) * TK;
            stage_k.fetch(kptr + (int64_t)k1 * p.sk.t, p.sk.t, p.T - k1, tid);
            stage_v.fetch(vptr + (int64_t)k1 * p.sv.t, p.sv.t, p.T - k1, tid);
        }
        if (kt < wr.start || kt >= wr.end) continue;
        const bool full = (kt >= wr.full_start) && (kt < wr.full_end);
        const int k0 = kt * TK;

        // S^T = K Q^T
        f32x16 s[KB];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s[kb][r] = 0.f;
            s[kb] = mma_rowwise<E, D>(lds_k, 32 * kb, qf, s[kb], lane);
        }

        float mx = -INFINITY;
        if (full) {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    s[kb][r] *= scale;
                    mx = fmaxf(mx, s[kb][r]);
                }
        } else {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    int key = k0 + 32 * kb + 8 * (r / 4) + 4 * h + (r % 4);
                    bool ok = (key < seq_len) && M::pred(q_pos, key, seq_len, p.margs);
                    s[kb][r] = ok ? s[kb][r] * scale : -INFINITY;
                    mx = fmaxf(mx, s[kb][r]);
                }
        }
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float pv = fast_exp2(s[kb][r] - m_safe);
                s[kb][r] = pv;
                psum += pv;
            }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= alpha;

        // O^T += V^T P^T
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int db = 0; db < DB; db++)
                o[db] = mma_transposed<E, D>(lds_v, 32 * kb, 32 * db, s[kb], o[db], lane);
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

// Launcher for one (element type, head dim); dispatches on the mask id and takes the tile shape
// from the static table.
template <typename E, int D>
int launch_fwd(const FwdParams& p, int mask_id, hipStream_t stream) {
    int status = CHILL_ERR_BAD_MASK;
    CHILL_DISPATCH_MASK(mask_id, {
        constexpr TileConfig cfg = fwd_tile_config(MASK_ID, D, Elem<E>::kDType);
        static_assert(cfg.rows == cfg.waves * 32, "one wave owns 32 rows");
        const int n_q_tiles = cdiv(p.T, cfg.rows);
        const int64_t total64 = (int64_t)p.B * p.H * n_q_tiles;
        if (total64 > ((int64_t)1 << 30)) return CHILL_ERR_TOO_LARGE;
        const int total = (int)total64;
        dim3 grid(cdiv(total, 8) * 8), block(cfg.waves * 64);
        auto kern = fwd_kernel<E, D, MASK_ID, cfg.waves, cfg.streamed>;
        const bool hfb = Mask<MASK_ID>::has_full_blocks(32, cfg.streamed, p.T, p.margs);
        if (cfg.lds_bytes > 48 * 1024) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, cfg.lds_bytes) != hipSuccess)
                return CHILL_ERR_HIP;
        }
        hipLaunchKernelGGL(kern, grid, block, cfg.lds_bytes, stream, p, n_q_tiles, total, hfb ? 1 : 0);
        status = (hipGetLastError() == hipSuccess) ? CHILL_OK : CHILL_ERR_HIP;
    });
    return status;
}

}  // namespace chill
