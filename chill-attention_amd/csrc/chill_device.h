// Device building blocks shared by the gfx950 attention kernels: MFMA wrappers per element type,
// the swizzled LDS tile format, cooperative global->LDS staging and the two A-operand readers
// (row-wise and transposed).
//
// Register layouts used throughout (64-lane wavefront, lane l, n = l % 32, h = l / 32):
//   * 32x32 MFMA accumulator, 16 floats c[r]:  element (row = 8*(r/4) + 4*h + r%4, col = n);
//   * 16-bit A/B operand of v_mfma_f32_32x32x16: 8 elements along the contraction axis,
//     lane (n, h) holds slots 8*h .. 8*h+7 of row/column n;
//   * fp32 A/B operand of v_mfma_f32_32x32x2: one element, lane (n, h) holds slot h.
// Because the contraction is a sum, any bijection between MFMA slots and real indices works as
// long as A and B agree.  That freedom lets an accumulator of a transposed product (keys on the
// rows) be fed back as a B operand with no cross-lane traffic:
//   * 16-bit: accumulator registers 8*s .. 8*s+7 (s = 0, 1) of a 32-row block are the 8 slots of
//     lane half h for the 16 rows {16*s + 8*(e/4) + 4*h + e%4, e = 0..7};
//   * fp32: accumulator register r is slot h for row 8*(r/4) + 4*h + r%4.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "chill_mask.h"

namespace chill {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

constexpr float kLog2e = 1.4426950408889634f;

struct bf16_t {};
struct f16_t {};
struct f32_t {};

template <typename T>
struct Elem;

template <>
struct Elem<bf16_t> {
    typedef __bf16 type;
    static constexpr int kBytes = 2;
    static constexpr bool k16 = true;
    static constexpr int kDType = CHILL_BF16;
    __device__ __forceinline__ static f32x16 mma(i32x4 a, i32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ __forceinline__ static i32x4 pack8(f32x8 v) {
        return __builtin_bit_cast(i32x4, __builtin_convertvector(v, bf16x8));
    }
    __device__ __forceinline__ static i32x2 pack4(f32x4 v) {
        return __builtin_bit_cast(i32x2, __builtin_convertvector(v, bf16x4));
    }
    __device__ __forceinline__ static float to_float(type x) { return (float)x; }
};

template <>
struct Elem<f16_t> {
    typedef _Float16 type;
    static constexpr int kBytes = 2;
    static constexpr bool k16 = true;
    static constexpr int kDType = CHILL_F16;
    __device__ __forceinline__ static f32x16 mma(i32x4 a, i32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ __forceinline__ static i32x4 pack8(f32x8 v) {
        return __builtin_bit_cast(i32x4, __builtin_convertvector(v, f16x8));
    }
    __device__ __forceinline__ static i32x2 pack4(f32x4 v) {
        return __builtin_bit_cast(i32x2, __builtin_convertvector(v, f16x4));
    }
    __device__ __forceinline__ static float to_float(type x) { return (float)x; }
};

template <>
struct Elem<f32_t> {
    typedef float type;
    static constexpr int kBytes = 4;
    static constexpr bool k16 = false;
    static constexpr int kDType = CHILL_F32;
    // one 16-byte chunk = 4 contraction slots per lane half = 4 MFMA steps
    __device__ __forceinline__ static f32x16 mma(i32x4 a, i32x4 b, f32x16 c) {
        f32x4 af = __builtin_bit_cast(f32x4, a);
        f32x4 bf = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int t = 0; t < 4; t++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(af[t], bf[t], c, 0, 0, 0);
        return c;
    }
    __device__ __forceinline__ static float to_float(type x) { return x; }
};

// Exchange a value between lane l and lane l ^ 32 (v_permlane32_swap).
__device__ __forceinline__ float swap32(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    int lane_hi = (threadIdx.x & 32);
    // r[0]: lanes < 32 keep their own value, lanes >= 32 receive the partner's;
    // r[1]: lanes < 32 receive the partner's, lanes >= 32 keep their own.
    int other = lane_hi ? r[0] : r[1];
    return __builtin_bit_cast(float, other);
}
__device__ __forceinline__ float max_across_halves(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
}
__device__ __forceinline__ float sum_across_halves(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ------------------------------------------------------------------------------------------
// LDS tile: ROWS x D elements, addressed in 16-byte chunks.  Chunk (row, c) has linear index
// L = row * CH + c and lives at phys(L) = L with its low four bits XORed by the next four, a
// bijection inside every aligned group of 16 chunks (256 bytes).  Lanes that read the same chunk
// column of consecutive rows (the row-wise A operand) land in different banks.
// ------------------------------------------------------------------------------------------
template <typename E, int D>
struct LdsTile {
    static constexpr int CH = D * Elem<E>::kBytes / 16;  // chunks per row
    static_assert(CH >= 1, "row shorter than one chunk");

    __device__ __forceinline__ static int phys(int L) { return L ^ ((L >> 4) & 15); }
    __device__ __forceinline__ static int chunk_off(int row, int c) { return phys(row * CH + c) * 16; }
    // byte offset of element (row, col)
    __device__ __forceinline__ static int elem_off(int row, int col) {
        constexpr int EPC = 16 / Elem<E>::kBytes;  // elements per chunk
        return chunk_off(row, col / EPC) + (col % EPC) * Elem<E>::kBytes;
    }
    static constexpr int bytes(int rows) { return rows * D * Elem<E>::kBytes; }
};

// Cooperative staging of a ROWS x D tile: each thread owns chunks L = tid, tid + NT, ...
// `fetch` reads them from global memory into registers (rows >= row_limit read as zero),
// `commit` writes the registers to LDS.  Splitting the two lets the global loads of the next tile
// fly while the current one is being consumed.
template <typename E, int D, int ROWS, int NT>
struct TileStager {
    typedef LdsTile<E, D> L;
    static constexpr int TOTAL = ROWS * L::CH;
    static constexpr int PER_THREAD = (TOTAL + NT - 1) / NT;
    i32x4 regs[PER_THREAD];

    // base points at row 0 of the tile; row_stride in elements; rows_valid = number of rows of the
    // tile that exist in the tensor (may be <= 0 or > ROWS).
    __device__ __forceinline__ void fetch(const typename Elem<E>::type* base, int64_t row_stride,
                                          int rows_valid, int tid) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            int idx = tid + i * NT;
            int row = idx / L::CH;
            int c = idx % L::CH;
            i32x4 val = {0, 0, 0, 0};
            if ((TOTAL % NT == 0 || idx < TOTAL) && row < rows_valid) {
                val = *reinterpret_cast<const i32x4*>(
                    reinterpret_cast<const char*>(base + (int64_t)row * row_stride) + c * 16);
            }
            regs[i] = val;
        }
    }
    __device__ __forceinline__ void commit(char* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < PER_THREAD; i++) {
            int idx = tid + i * NT;
            if (TOTAL % NT == 0 || idx < TOTAL) {
                *reinterpret_cast<i32x4*>(lds + L::phys(idx) * 16) = regs[i];
            }
        }
    }
};

// Row-wise A/B operand: the 16-byte chunk (row, 2*j + h).  For 16-bit types that is one MFMA
// operand (contraction slots 16*j + 8*h ..), for fp32 four of them (slots 8*j + 4*h ..).
template <typename E, int D>
__device__ __forceinline__ i32x4 lds_row_chunk(const char* lds, int row, int c) {
    return *reinterpret_cast<const i32x4*>(lds + LdsTile<E, D>::chunk_off(row, c));
}

// Transposed A operand for 16-bit types, built from two ds_read_b64_tr_b16.
// That instruction works on groups of 16 lanes: lane r of a group supplies the address of four
// consecutive 16-bit elements X[k0 + r/4][n0 + 4*(r%4) ..], and lane i of the group receives
// X[k0 + 0..3][n0 + i].  Here: rows = contraction index (4 consecutive rows per read), the wave's
// 32 output rows n split into two groups of 16 columns.
// Returns the operand for rows {row0 + 4*h + (0..3), row0 + 8 + 4*h + (0..3)} at column col0 + n.
template <typename E, int D>
__device__ __forceinline__ i32x4 lds_tr_operand(const char* lds, int row0, int col0, int lane) {
    typedef LdsTile<E, D> L;
    int h = lane >> 5;
    int r = lane & 15;
    int colgrp = (lane >> 4) & 1;
    int col = col0 + 16 * colgrp + 4 * (r & 3);
    if (D < 32) col &= (D - 1);
    int row = row0 + 4 * h + (r >> 2);
    const lds_i16x4* p0 = (const lds_i16x4*)(lds + L::elem_off(row, col));
    const lds_i16x4* p1 = (const lds_i16x4*)(lds + L::elem_off(row + 8, col));
    i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)p0);
    i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)p1);
    i16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(i32x4, v);
}

// acc(32 out-rows x 32 cols) += X^T(rows of the LDS tile [row0, row0+32) as contraction) * P,
// where P is a 32x32 accumulator-layout block (rows = contraction index) reused as B operand.
// Output row index = column of the LDS tile (col0 + n).
template <typename E, int D>
__device__ __forceinline__ f32x16 mma_transposed(const char* lds, int row0, int col0, f32x16 p,
                                                 f32x16 acc, int lane) {
    if constexpr (Elem<E>::k16) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            f32x8 ps;
#pragma unroll
            for (int e = 0; e < 8; e++) ps[e] = p[8 * s + e];
            i32x4 b = Elem<E>::pack8(ps);
            i32x4 a = lds_tr_operand<E, D>(lds, row0 + 16 * s, col0, lane);
            acc = Elem<E>::mma(a, b, acc);
        }
    } else {
        typedef LdsTile<E, D> L;
        int h = lane >> 5;
        int col = col0 + (lane & 31);
        if (D < 32) col &= (D - 1);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int row = row0 + 8 * (r / 4) + 4 * h + (r % 4);
            float a = *reinterpret_cast<const float*>(lds + L::elem_off(row, col));
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, p[r], acc, 0, 0, 0);
        }
    }
    return acc;
}

// acc(32 rows of the LDS tile x 32 cols) += X[row0 + 0..31][:] * B^T where the B operand chunks
// (resident rows, e.g. the wave's Q rows) live in registers: b.c[j] = chunk (n, 2*j + h).
template <typename E, int D>
struct Resident {
    static constexpr int NJ = LdsTile<E, D>::CH / 2;
    static_assert(NJ >= 1, "head dim too small");
    i32x4 c[NJ];
};

template <typename E, int D>
__device__ __forceinline__ f32x16 mma_rowwise(const char* lds, int row0, const Resident<E, D>& b,
                                              f32x16 acc, int lane) {
    constexpr int NJ = Resident<E, D>::NJ;
    int n = lane & 31, h = lane >> 5;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        i32x4 a = lds_row_chunk<E, D>(lds, row0 + n, 2 * j + h);
        acc = Elem<E>::mma(a, b.c[j], acc);
    }
    return acc;
}

// Load the resident operand chunks of the wave's 32 rows straight from global memory:
// regs[j] = 16 bytes at (row n, chunk 2*j + h); rows >= rows_valid read as zero.
template <typename E, int D>
__device__ __forceinline__ void load_resident(Resident<E, D>& regs,
                                              const typename Elem<E>::type* base, int64_t row_stride,
                                              int rows_valid, int lane) {
    constexpr int NJ = Resident<E, D>::NJ;
    int n = lane & 31, h = lane >> 5;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        i32x4 val = {0, 0, 0, 0};
        if (n < rows_valid) {
            val = *reinterpret_cast<const i32x4*>(
                reinterpret_cast<const char*>(base + (int64_t)n * row_stride) + (2 * j + h) * 16);
        }
        regs.c[j] = val;
    }
}

// Store one output row from transposed accumulators: lane (n, h) holds, for every 32-wide block
// db of the head dim, the 16 values of columns d = 32*db + 8*(r/4) + 4*h + r%4 of ITS row.
// Each group of four consecutive r is four consecutive d, written as one 8- or 16-byte store.
// Rows that are not `valid` are written as zeros.
template <typename E, int D>
__device__ __forceinline__ void store_row_transposed(typename Elem<E>::type* row_ptr,
                                                     const f32x16 (&acc)[(D + 31) / 32], float mult,
                                                     bool valid, int h) {
    constexpr int DB = (D + 31) / 32;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            int d0 = 32 * db + 8 * g + 4 * h;
            if (D >= 32 || d0 < D) {
                f32x4 vals;
#pragma unroll
                for (int e = 0; e < 4; e++) vals[e] = valid ? acc[db][4 * g + e] * mult : 0.f;
                if constexpr (Elem<E>::k16) {
                    *reinterpret_cast<i32x2*>(row_ptr + d0) = Elem<E>::pack4(vals);
                } else {
                    *reinterpret_cast<f32x4*>(row_ptr + d0) = vals;
                }
            }
        }
}

// Zero rows [row0, row0 + nrows) of a [T, D] slab (inner stride 1) cooperatively.
template <typename E, int D, int NT>
__device__ __forceinline__ void zero_rows(typename Elem<E>::type* base, int64_t row_stride, int row0,
                                          int nrows, int tid) {
    constexpr int CH = LdsTile<E, D>::CH;
    const i32x4 z = {0, 0, 0, 0};
    for (int idx = tid; idx < nrows * CH; idx += NT) {
        int row = row0 + idx / CH;
        int c = idx % CH;
        *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(base + (int64_t)row * row_stride) + c * 16) = z;
    }
}

// Work-item order: workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so the
// linear workgroup id is remapped to give every XCD a contiguous run of work items.  Returns the
// work item index or -1 when this workgroup has nothing to do.
__device__ __forceinline__ int xcd_contiguous_item(int wg, int total) {
    constexpr int kXcds = 8;
    int per = (total + kXcds - 1) / kXcds;
    int item = (wg % kXcds) * per + wg / kXcds;
    return (wg / kXcds < per && item < total) ? item : -1;
}

}  // namespace chill
