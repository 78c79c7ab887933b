// Forward kernel with O^T in hand-managed accumulation registers (16-bit inputs, wide rows).
//
// Same algorithm, LDS staging and tile decisions as fwd_q_tile (chill_fwd_kernel.h): 4 waves, one per
// SIMD, 32 query rows each, Q^T resident as MFMA B operands, S^T = K Q^T per 32-key step, lazy
// online-softmax rescale, O^T += V^T P^T through the transposing LDS read (chill_fwd.py:21-359).
// At D = 256 the resident Q takes 64 registers and O^T 128; left to the compiler, parts of O^T travel
// between the two register files in every step.  Here O^T sits in the accumulation registers under
// fixed names (see the hand-placed MFMA helpers in chill_device.h); the rare rescale is the only
// other code that touches it.
// Included by chill_fwd_kernel.h (between fwd_q_tile and the launcher), not on its own.
#pragma once

namespace chill {

// a[BASE .. BASE+15] *= alpha (rare path of the lazy softmax rescale)
template <int BASE>
__device__ __forceinline__ void agpr_scale_block(float alpha, int& tok) {
    static_for<16>([&](auto e) {
        float x;
        asm volatile("v_accvgpr_read_b32 %0, a[%2]" : "=v"(x), "+v"(tok) : "n"(BASE + e));
        x *= alpha;
        asm volatile("v_accvgpr_write_b32 a[%1], %2" : "+v"(tok) : "n"(BASE + e), "v"(x));
    });
}

// One q-tile (128 query rows of one head) from start to finish.
template <typename E, int D, int MASK, int TK, int NS>
__device__ __forceinline__ void fwd_q_tile_regs(const FwdParams& p, char* smem, int b, int hd, int qt,
                                                int wave_has_full_blocks) {
    using ET = typename Elem<E>::type;
    using M = Mask<MASK>;
    // guarded softmax (see fwd_kernel): not for the banded masks, whose rows end after a few blocks
    constexpr bool kGuard = !mask_is_banded(MASK);
    constexpr float kGuardLimit = Elem<E>::kDType == CHILL_F16 ? 32768.f : 1.0e18f;
    static_assert(Elem<E>::k16, "16-bit element types");
    typedef FwdLds<E, D, TK> Lds;
    typedef typename Lds::KT KT;
    typedef typename Lds::VT VT;
    constexpr int NW = 4;
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
    const int ta = wr.start - wg.start, tb = wr.end - wg.start;
    const int fa = wr.full_start - wg.start, fb = wr.full_end - wg.start;

    // per-lane LDS offsets inside a stage; everything else is an immediate
    const int k_lane = n * KT::PITCH + h * 16;
    int v_lane;
    {
        const int r = lane & 15, colgrp = (lane >> 4) & 1;
        const int col = 16 * colgrp + 4 * (r & 3);
        v_lane = Lds::K_BYTES + (4 * h + (r >> 2)) * VT::PITCH + col * 2;
    }

    // O^T block db lives in a[O_BASE + 16 * db ..], at the top of the file
    constexpr int O_BASE = 256 - 16 * DB;
    static_assert(O_BASE >= 0, "accumulators exceed the accumulation registers");
    int tok = agpr_zero<O_BASE, 16 * DB>();
    float m_run = -INFINITY;  // reference max of the row (scaled, log2 domain)
    float m_use = 0.f;        // m_run, or 0 while the row has seen no unmasked key
    float l_run = 0.f;        // this lane's share of the row sum
    const int q_pos = qw + n;
    const Range vis = visible_range<MASK, true>(q_pos, seq_len, p.margs);  // the keys this lane's row sees
    // A negative scale reverses the order of the scores: the sign goes into Q, the softmax works
    // with |scale| (max(scale * s) = |scale| * max(sign * s)).
    const float scale = fabsf(p.scale_log2);

    // S^T block of step kb: K[32 rows][:] Q^T
    auto scores = [&](f32x16& dst, const lds_char* stage, int kb) {
        const lds_char* base = stage + k_lane + kb * 32 * KT::PITCH;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const i32x4 a = *reinterpret_cast<const lds_i32x4*>(base + j * 32);
            if (j == 0)
                Mfma16<E>::set(a, qf.c[j], dst, tok);
            else
                Mfma16<E>::add(a, qf.c[j], dst, tok);
        }
    };
    // mask and block max (scaled) of a score block whose MFMAs have been issued
    auto prepare = [&](f32x16& sc, bool full, int key0) -> float {
        mfma_fence(sc);
        if (!full) {
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
        }
        if constexpr (kGuard) return 0.f;  // no block max on the common path
        float mx = sc[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, sc[r]);
        return max_across_halves(mx) * scale;
    };
    // O^T += V^T P^T for step kb: one packed P operand per 16 keys feeds all head-dim blocks
    auto accumulate = [&](const i32x4 (&bop)[2], const lds_char* stage, int kb) {
        const lds_char* base = stage + v_lane + kb * 32 * VT::PITCH;
        static_for<2>([&](auto s2) {
            static_for<DB>([&](auto db) {
                const lds_char* a0 = base + (16 * s2) * VT::PITCH + db * 64;
                const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)a0);
                const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(a0 + 8 * VT::PITCH));
                const i32x4 a = __builtin_bit_cast(i32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                Mfma16<E>::template acc<O_BASE + 16 * db>(a, bop[s2], tok);
            });
        });
    };

    f32x16 s[2];         // scores of the current and of the next step
    float mx_cur = 0.f;  // block max of s[current], already scaled
    float guard_above = -1.f;
    const lds_char* lds0 = (const lds_char*)smem;
    // Q must have arrived before the loop: inside it the only vector-memory traffic is the async
    // tile loads, and the compiler must not place a wait for them in front of the first MFMA
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (p.scale_log2 < 0.f) {
#pragma unroll
            for (int e = 0; e < 4; e++) qf.c[j][e] ^= (int)0x80008000;
        }
        asm volatile("" ::"v"(qf.c[j]));
    }

    // One step: softmax of the current 32-key block and its share of O, with the scores of the next
    // block of the tile issued first.
    auto step = [&](const lds_char* stage, int kb, bool full, int k0) {
        f32x16& cur = s[kb & 1];
        f32x16& nxt = s[(kb + 1) & 1];
        // raise the reference max of the lanes in `raise` to at least m_block and rescale what has been accumulated
        auto raise_reference = [&](bool raise, float m_block) {
            // the accumulating MFMAs of the previous step must have left the pipeline
            asm volatile("s_nop 15\n\ts_nop 15" : "+v"(tok));
            const float m_new = raise ? fmaxf(m_run, m_block) : m_run;
            const float m_use_new = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_use - m_use_new);
            m_run = m_new;
            m_use = m_use_new;
            l_run *= alpha;
            static_for<DB>([&](auto db) { agpr_scale_block<O_BASE + 16 * db>(alpha, tok); });
            asm volatile("s_nop 3" : "+v"(tok));
        };
        if constexpr (!kGuard) {
            // rare path: the block max computed in the previous step exceeds the reference by more than tau
            const bool raise = mx_cur > m_run + kRescaleTau;
            if (__builtin_amdgcn_ballot_w64(raise) != 0) raise_reference(raise, mx_cur);
        }
        const bool have_next = kb + 1 < KB;
        // scores of the next step fly while this step's softmax runs
        if (have_next) scores(nxt, stage, kb + 1);
        float psum = 0.f;
        i32x4 pb[2];
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
        if constexpr (kGuard) {
            // Guarded softmax, as in fwd_kernel: a row keeps the max of its first visible block as reference
            // while the block sums stay below guard_above; a row without reference has guard_above = -1.
            const unsigned long long fired = __builtin_amdgcn_ballot_w64(psum > guard_above);
            if (fired != 0) {
                // the two lanes of a row (l and l ^ 32) hold half of its keys each and share its reference
                const bool fire = (((fired | (fired >> 32) | (fired << 32)) >> lane) & 1) != 0;
                float mx = cur[0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, cur[r]);
                raise_reference(fire, max_across_halves(mx) * scale);
                guard_above = (m_run == -INFINITY) ? -1.f : kGuardLimit;
                softmax_block();
            }
        }
        l_run += psum;
        accumulate(pb, stage, kb);
        if (have_next) mx_cur = prepare(nxt, full, k0 + 32 * (kb + 1));
    };

    int st_cur = NS - 1;  // LDS stage of tile i (advanced at the top of the loop)
    int st_issue = LA;    // LDS stage the next issued tile goes to
    for (int i = 0; i < n_tiles; i++) {
        // tile i has landed for every wave (the newer ones may still be in flight: every wave issues at
        // least TILE_LOADS loads per full tile, and the tiles behind tile i are full ones while another
        // tile follows them), and everyone is done with tile i - 1
        constexpr int TILE_LOADS = decltype(load_k)::SLABS / NW + decltype(load_v)::SLABS / NW;
        if (LA > 0 && i + LA < n_tiles - 1)
            wait_async_tiles_except<LA * TILE_LOADS>();
        else
            wait_async_tiles();
        __syncthreads();
        st_cur = st_cur + 1 == NS ? 0 : st_cur + 1;
        st_issue = st_issue + 1 == NS ? 0 : st_issue + 1;
        if (i + LA + 1 < n_tiles) issue_tile(i + LA + 1, st_issue);
        if (i < ta || i >= tb) continue;
        const lds_char* stage = lds0 + st_cur * Lds::STAGE_BYTES;
        const bool full = (i >= fa) && (i < fb);
        const int k0 = (wg.start + i) * TK;
        scores(s[0], stage, 0);
        mx_cur = prepare(s[0], full, k0);
#pragma unroll
        for (int kb = 0; kb < KB; kb++) step(stage, kb, full, k0);
    }

    // epilogue: O = acc / l, LSE2 = m + log2(l) (chill_fwd.py:288-289, 327-328)
    agpr_drain(tok);
    f32x16 o[DB];
    static_for<DB>([&](auto db) { o[db] = agpr_read_block<O_BASE + 16 * db>(); });
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

// The workgroup-to-q-tile mapping of fwd_kernel (pairs of q-tiles, or one each).
template <typename E, int D, int MASK, int TK, int NS>
__global__ __launch_bounds__(256) void fwd_regs_kernel(FwdParams p, int n_q_tiles, int total_items,
                                                      int wave_has_full_blocks, int paired) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int item = xcd_contiguous_item(blockIdx.x, total_items);
    if (item < 0) return;
    agpr_reserve();
    const int per_head = paired ? (n_q_tiles + 1) / 2 : n_q_tiles;
    const int bh = item / per_head;
    const int j = item % per_head;
    const int b = bh / p.H;
    const int hd = bh % p.H;
    const int qt_hi = n_q_tiles - 1 - j;
    fwd_q_tile_regs<E, D, MASK, TK, NS>(p, smem, b, hd, qt_hi, wave_has_full_blocks);
    if (paired && j != qt_hi) {
        __syncthreads();  // the LDS ring is reused
        fwd_q_tile_regs<E, D, MASK, TK, NS>(p, smem, b, hd, j, wave_has_full_blocks);
    }
#ifdef CHILL_TEST_UNSOUND_REGISTERS
    // For the test of the build's register check only: the COMPILER reads an accumulation register here,
    // which a kernel that manages a128..a255 by itself must never let happen.
    float from_accumulation_register;
    asm volatile("v_accvgpr_write_b32 %0, 0" : "=a"(from_accumulation_register));
    if (p.lse != nullptr && p.T < 0) p.lse[0] = from_accumulation_register;
#endif
}

}  // namespace chill
