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

#include <utility>

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
typedef __attribute__((address_space(3))) i32x4 lds_i32x4;
typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) float lds_float;

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
    __device__ __forceinline__ static int pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(int, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
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
    __device__ __forceinline__ static int pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(int, __builtin_convertvector(f32x2{lo, hi}, f16x2));
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

// A value that is the same in every lane, in a scalar register (says so where the compiler has lost track:
// an "s" operand of an inline-asm statement must be one).
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ unsigned uniform(unsigned x) { return (unsigned)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ float uniform(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}
template <typename T>
__device__ __forceinline__ const T* uniform(const T* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = uniform((unsigned)v), hi = uniform((unsigned)(v >> 32));
    return (const T*)(((unsigned long long)hi << 32) | lo);
}

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

// ------------------------------------------------------------------------------------------
// Hand-placed MFMAs (16-bit types).  A kernel that runs one wave per SIMD owns 512 registers per
// lane: 256 ordinary ones, which the compiler allocates, and the 256 accumulation registers
// a0..a255, which such a kernel manages by itself: blocks that only MFMAs touch for a whole loop
// live there under fixed names, out of the compiler's sight (given the choice, the compiler moves a
// block between the two files around every use).  Rules for a kernel that uses these helpers:
//   * it calls agpr_reserve() first (declares a0..a255 used, so the wave gets all 512 registers);
//   * it names its blocks from a255 downwards: a compiler that runs out of ordinary registers parks
//     values in the lowest accumulation registers.  Whether it stayed below the hand-named ones is
//     checked on the assembly of every build that instantiates such a kernel
//     (chill_attention/tune.py, hand_managed_registers);
//   * it contains no MFMA builtin (their results would be routed through the same registers);
//   * the compiler does not see the latency of these instructions: mfma_fence() stands between
//     the last MFMA that writes a block of ordinary registers and the first other instruction that
//     reads it, agpr_drain() between the last accumulating MFMA and agpr_read_block().
// Fences, drains and register reads are volatile asm statements; the MFMAs keep their program order
// through a token (below).
// ------------------------------------------------------------------------------------------
#define CHILL_A10(b) "a" #b "0", "a" #b "1", "a" #b "2", "a" #b "3", "a" #b "4", "a" #b "5", "a" #b "6", "a" #b "7", "a" #b "8", "a" #b "9"
__device__ __forceinline__ void agpr_reserve() {
    asm volatile("" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", CHILL_A10(1), CHILL_A10(2), CHILL_A10(3),
                 CHILL_A10(4), CHILL_A10(5), CHILL_A10(6), CHILL_A10(7), CHILL_A10(8), CHILL_A10(9), CHILL_A10(10),
                 CHILL_A10(11), CHILL_A10(12), CHILL_A10(13), CHILL_A10(14), CHILL_A10(15), CHILL_A10(16), CHILL_A10(17),
                 CHILL_A10(18), CHILL_A10(19), CHILL_A10(20), CHILL_A10(21), CHILL_A10(22), CHILL_A10(23), CHILL_A10(24),
                 "a250", "a251", "a252", "a253", "a254", "a255");
}
#undef CHILL_A10

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{})
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

template <int I>
__device__ __forceinline__ void agpr_zero_one() {
    asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(I));
}
template <int BASE, int... I>
__device__ __forceinline__ void agpr_zero_seq(std::integer_sequence<int, I...>) {
    (agpr_zero_one<BASE + I>(), ...);
}
// a[BASE .. BASE + N - 1] = 0; returns the token the accumulating MFMAs are chained on
template <int BASE, int N>
__device__ __forceinline__ int agpr_zero() {
    agpr_zero_seq<BASE>(std::make_integer_sequence<int, N>{});
    int tok;
    asm volatile("v_mov_b32 %0, 0" : "=v"(tok));
    return tok;
}

template <int I>
__device__ __forceinline__ float agpr_read_one() {
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(I));
    return x;
}
template <int BASE, int... I>
__device__ __forceinline__ f32x16 agpr_read_seq(std::integer_sequence<int, I...>) {
    f32x16 r;
    ((r[I] = agpr_read_one<BASE + I>()), ...);
    return r;
}
// the 32x32 accumulator block held in a[BASE .. BASE + 15]
template <int BASE>
__device__ __forceinline__ f32x16 agpr_read_block() {
    return agpr_read_seq<BASE>(std::make_integer_sequence<int, 16>{});
}
__device__ __forceinline__ void agpr_drain(int tok) { asm volatile("s_nop 15\n\ts_nop 15" ::"v"(tok) : "memory"); }

// `tok` threads a data dependency through the MFMAs: it keeps them in program order, and the
// accumulating ones (which have no other output the compiler can see) alive, without making them
// volatile (LDS reads may not move across a volatile asm statement, and each one would then expose its
// full latency).  A chain of MFMAs that accumulate into one block may be issued back to back (the
// hardware forwards the block); callers that have two independent chains alternate between them all the
// same.  The chain of tokens starts at agpr_zero() and ends in agpr_drain().
template <typename E>
struct Mfma16;
#define CHILL_MFMA16(TYPE, MNEMONIC)                                                                          \
    template <>                                                                                               \
    struct Mfma16<TYPE> {                                                                                     \
        /* a[BASE .. BASE+15] += A B; an operand written by the vector ALU just before needs the 2 wait states */ \
        template <int BASE>                                                                                   \
        __device__ __forceinline__ static void acc(i32x4 a, i32x4 b, int& tok) {                              \
            asm("s_nop 1\n\t" MNEMONIC " a[%3:%4], %1, %2, a[%3:%4]"                                          \
                : "+v"(tok) : "v"(a), "v"(b), "n"(BASE), "n"(BASE + 15));                                     \
        }                                                                                                     \
        /* c = A B and c += A B with c in ordinary registers */                                               \
        __device__ __forceinline__ static void set(i32x4 a, i32x4 b, f32x16& c, int& tok) {                   \
            asm(MNEMONIC " %0, %2, %3, 0" : "=&v"(c), "+v"(tok) : "v"(a), "v"(b));                            \
        }                                                                                                     \
        __device__ __forceinline__ static void add(i32x4 a, i32x4 b, f32x16& c, int& tok) {                   \
            asm(MNEMONIC " %0, %2, %3, %0" : "+v"(c), "+v"(tok) : "v"(a), "v"(b));                            \
        }                                                                                                     \
    };
CHILL_MFMA16(bf16_t, "v_mfma_f32_32x32x16_bf16")
CHILL_MFMA16(f16_t, "v_mfma_f32_32x32x16_f16")
#undef CHILL_MFMA16

// An 8-pass MFMA needs 11 wait states before another kind of instruction may read its result.
__device__ __forceinline__ void mfma_fence(f32x16& x0, f32x16& x1, f32x16& x2, f32x16& x3) {
    asm volatile("s_nop 11" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
}
__device__ __forceinline__ void mfma_fence(f32x16& x0, f32x16& x1) {
    asm volatile("s_nop 11" : "+v"(x0), "+v"(x1));
}
__device__ __forceinline__ void mfma_fence(f32x16& x0) { asm volatile("s_nop 11" : "+v"(x0)); }

// Masking a 32 x 32 accumulator block by a range.  A lane holds, for its own row (or column) of the
// block, the 16 entries at positions pos0 + 8 * (r / 4) + (r % 4) of the other axis, where pos0 = first
// position of the block + 4 * (lane / 32).  Entries outside [lo, hi] become `fill`.  Most partial
// blocks are cut on one side only (wave-uniform test), which leaves one comparison per entry.
__device__ __forceinline__ void fill_outside_range(f32x16& s, int lo, int hi, int pos0, float fill) {
    const int a = lo - pos0, b = hi - pos0;  // entry r is visible iff a <= c(r) <= b, c(r) = 8 * (r / 4) + (r % 4)
    if (__builtin_amdgcn_ballot_w64(a > 0) == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = (8 * (r / 4) + (r % 4) <= b) ? s[r] : fill;
    } else if (__builtin_amdgcn_ballot_w64(b < 27) == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = (8 * (r / 4) + (r % 4) >= a) ? s[r] : fill;
    } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int c = 8 * (r / 4) + (r % 4);
            s[r] = (c >= a && c <= b) ? s[r] : fill;
        }
    }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ------------------------------------------------------------------------------------------
// LDS tile: ROWS x D elements, addressed in 16-byte chunks.  Chunk (row, c) has linear index
// L = row * CH + c and lives at phys(L) = L ^ g(key), where key is the index of the 256-byte line
// (of the row, for rows longer than a line) and g swaps the two 2-bit halves of key & 15.  The XOR
// only touches the low four bits of L, so it is an involution inside every aligned group of 16
// chunks.  Measured on gfx950 (64 banks x 4 B; a 16-byte read serves 16 lanes per cycle, an 8-byte
// read 32 lanes per cycle) both access patterns of the kernels are conflict-free with it:
//   * row-wise operand: 16 consecutive rows, same chunk column -> g(key) takes 16 values;
//   * transposed operand: 4 consecutive rows x 64 contiguous bytes -> bits 2..3 of g(key), the
//     64-byte segment index, take 4 values.
// ------------------------------------------------------------------------------------------
template <typename E, int D>
struct LdsTile {
    static constexpr int CH = D * Elem<E>::kBytes / 16;  // chunks per row
    static_assert(CH >= 2, "row shorter than two chunks");
    static constexpr int BLOCK_BYTES = 32 * CH * 16;     // 32 rows
    // +32 rows leaves the swizzle key unchanged (mod 16) when 32 rows are a multiple of 16 lines
    static constexpr bool kBlockAffine = CH >= 8;

    __device__ __forceinline__ static int swz(int t) { return ((t & 3) << 2) | ((t >> 2) & 3); }
    __device__ __forceinline__ static int phys(int L) { return L ^ swz(CH > 16 ? (L >> 5) : (L >> 4)); }
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

// One asynchronous 16-byte global->LDS copy per lane: lane l's data lands at lds_base + 16*l.
// Written as inline asm so the compiler does not serialise later LDS reads behind it; the caller
// orders things with wait_async_tiles() + a workgroup barrier.  lds_base must be wave-uniform.
__device__ __forceinline__ void async_load16(const void* tile_base, int byte_off, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base), "v"(byte_off), "s"(tile_base) : "memory");
}

// Same for one 4-byte value per lane (lane l's value lands at lds_base + 4*l).
__device__ __forceinline__ void async_load4(const void* base, int byte_off, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_base), "v"(byte_off), "s"(base) : "memory");
}

__device__ __forceinline__ unsigned lds_address(const void* p) {
    return (unsigned)(unsigned long long)(const __attribute__((address_space(3))) char*)p;
}

// Asynchronous staging of a ROWS x D tile into a swizzled LdsTile (tiles that are read both
// row-wise and transposed).  One wave instruction fills a 1 KiB slab: lane l's 16 bytes land at
// slab base + 16*l, so the lane FETCHES the logical chunk whose swizzled position is its slot (the
// swizzle is an involution).  Rows >= rows_valid are zero-filled with ordinary LDS stores.  The
// caller waits with wait_async_tiles() and then a workgroup barrier before anyone reads the tile.
template <typename E, int D, int ROWS, int NT>
struct AsyncSwizzledLoader {
    typedef LdsTile<E, D> L;
    static constexpr int SLOTS = ROWS * L::CH;  // a multiple of 64
    static constexpr int SLABS = SLOTS / 64;
    static constexpr int NWV = NT / 64;
    static constexpr int PER_WAVE = (SLABS + NWV - 1) / NWV;
    static_assert(SLOTS % 64 == 0, "tile must be a whole number of 1 KiB slabs");
    int goff[PER_WAVE];  // byte offset of this lane's chunk from the tile's first row

    __device__ __forceinline__ void init(int64_t row_stride, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            int lg = L::phys((i * NWV + wave) * 64 + lane);
            goff[i] = (int)((lg / L::CH) * row_stride * Elem<E>::kBytes) + (lg % L::CH) * 16;
        }
    }

    __device__ __forceinline__ void issue(const typename Elem<E>::type* tile_base, int rows_valid, char* lds,
                                          int wave, int lane) const {
        const unsigned lds_base = lds_address(lds);
        if (rows_valid >= ROWS) {
#pragma unroll
            for (int i = 0; i < PER_WAVE; i++) {
                const int slab = i * NWV + wave;
                if (SLABS % NWV != 0 && slab >= SLABS) continue;
                async_load16(tile_base, goff[i], lds_base + slab * 1024);
            }
        } else {
#pragma unroll
            for (int i = 0; i < PER_WAVE; i++) {
                const int slab = i * NWV + wave;
                if (SLABS % NWV != 0 && slab >= SLABS) continue;
                int slot = slab * 64 + lane;
                int row = L::phys(slot) / L::CH;
                if (row < rows_valid) {
                    async_load16(tile_base, goff[i], lds_base + slab * 1024);
                } else {
                    *reinterpret_cast<i32x4*>(lds + slot * 16) = i32x4{0, 0, 0, 0};
                }
            }
        }
    }
};

// All asynchronous tile loads issued so far by this wave have landed in LDS.
__device__ __forceinline__ void wait_async_tiles() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// All but the N most recent vector-memory operations of this wave have completed (loads complete in
// issue order).  For a ring that keeps tiles in flight beyond the one about to be consumed: N = the
// number of loads the wave issued for those newer tiles, or less.
template <int N>
__device__ __forceinline__ void wait_async_tiles_except() {
    static_assert(N >= 0 && N <= 63, "the counter has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// ------------------------------------------------------------------------------------------
// Padded LDS tile: rows of D elements at a pitch of RB + PAD bytes.  Addresses are affine in
// (row, column), so every LDS read of the inner loops is "per-lane base register + immediate".
// Used where a tile is read in one pattern only (forward: K row-wise, V transposed); the pad is
// chosen per pattern (measured on gfx950, 64 banks x 4 B):
//   * row-wise 16-byte reads (16 lanes = 16 consecutive rows per cycle): PAD = 16;
//   * transposed 8-byte reads (32 lanes = 4 consecutive rows x 64 bytes per cycle): pitch = 64 mod 256;
//   * fp32 column reads (two rows four apart per cycle): pitch = 32 mod 64.
// ------------------------------------------------------------------------------------------
template <typename E, int D, int PAD>
struct PaddedTile {
    static constexpr int RB = D * Elem<E>::kBytes;
    static constexpr int CH = RB / 16;
    static constexpr int PITCH = RB + PAD;
    static constexpr int CHP = PITCH / 16;  // 16-byte slots per row, padding included
    static_assert(PAD % 16 == 0, "pad in whole chunks");
    static constexpr int bytes(int rows) { return rows * PITCH; }
};

template <typename E, int D>
constexpr int rowwise_pad() { return 16; }
template <typename E, int D>
constexpr int transposed_pad() {
    return Elem<E>::k16 ? (D * Elem<E>::kBytes >= 128 ? 64 : 0) : 32;
}

// Asynchronous staging of a ROWS x D tile into a PaddedTile.  Each wave instruction fills one
// 1 KiB slab; a lane's slot maps to (row, chunk) = (slot / CHP, slot % CHP).
// The per-lane global offsets are computed once (init) because the tile geometry never changes.
template <typename E, int D, int PAD, int ROWS, int NT>
struct AsyncPaddedLoader {
    typedef PaddedTile<E, D, PAD> P;
    static constexpr int SLOTS = ROWS * P::CHP;
    static constexpr int SLABS = (SLOTS + 63) / 64;
    static constexpr int NWV = NT / 64;
    static constexpr int PER_WAVE = (SLABS + NWV - 1) / NWV;
    static constexpr bool kPartialLastSlab = SLOTS % 64 != 0;
    // byte offset from the tile's first row.  Pad slots fetch (harmlessly) the first chunk of
    // their row, so a full tile needs no lane masking; -1 marks slots past the end of the tile.
    int goff[PER_WAVE];

    __device__ __forceinline__ void init(int64_t row_stride, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            int slot = (i * NWV + wave) * 64 + lane;
            int row = slot / P::CHP, c = slot % P::CHP;
            goff[i] = slot < SLOTS ? (int)(row * row_stride * Elem<E>::kBytes) + (c < P::CH ? c * 16 : 0) : -1;
        }
    }

    // tile_base: global address of the tile's first row (wave-uniform); lds: the tile in LDS.
    __device__ __forceinline__ void issue(const typename Elem<E>::type* tile_base, int64_t row_stride,
                                          int rows_valid, char* lds, int wave, int lane) const {
        const unsigned lds_base = lds_address(lds);
        if (rows_valid >= ROWS) {
#pragma unroll
            for (int i = 0; i < PER_WAVE; i++) {
                const int slab = i * NWV + wave;
                if (SLABS % NWV != 0 && slab >= SLABS) continue;
                if (kPartialLastSlab && (i + 1) * NWV >= SLABS) {
                    if (goff[i] >= 0) async_load16(tile_base, goff[i], lds_base + slab * 1024);
                } else {
                    async_load16(tile_base, goff[i], lds_base + slab * 1024);
                }
            }
        } else {
            // ragged last tile: rows past the end of the tensor read as zeros
#pragma unroll
            for (int i = 0; i < PER_WAVE; i++) {
                const int slab = i * NWV + wave;
                if (SLABS % NWV != 0 && slab >= SLABS) continue;
                int slot = slab * 64 + lane;
                int row = slot / P::CHP, c = slot % P::CHP;
                if (slot < SLOTS && c < P::CH) {
                    if (row < rows_valid) {
                        async_load16(tile_base, goff[i], lds_base + slab * 1024);
                    } else {
                        *reinterpret_cast<i32x4*>(lds + slot * 16) = i32x4{0, 0, 0, 0};
                    }
                }
            }
        }
    }
};

// Resident operand: the wave's 32 rows as MFMA B operands in registers,
// c[j] = the 16-byte chunk (row n, 2*j + h).
template <typename E, int D>
struct Resident {
    static constexpr int NJ = LdsTile<E, D>::CH / 2;
    static_assert(NJ >= 1, "head dim too small");
    i32x4 c[NJ];
};

// Per-lane byte offsets of everything a wave reads from a swizzled LdsTile, computed once per
// kernel; inside the loops an LDS address is "tile base + lane offset" plus an immediate.
// Offsets are for the first 32-row block of a tile; block kb adds kb * BLOCK_BYTES (valid when
// LdsTile::kBlockAffine, otherwise the address is recomputed).
//   row[j]          16-byte chunk (row n, 2*j + h): the row-wise operand.  For 16-bit types one
//                   MFMA operand (contraction slots 16*j + 8*h ..), for fp32 four (slots 8*j + 4*h ..).
//   tr[db][s][w]    16-bit types: address this lane supplies to ds_read_b64_tr_b16 for the transposed
//                   operand of head-dim block db, 16-row half s, first (w = 0) or second (w = 1)
//                   group of four contraction rows.  When 16 rows are a whole number of swizzle
//                   periods only s = 0 is stored and s = 1 is 16 rows further.
// ds_read_b64_tr_b16 works on groups of 16 lanes: lane r of a group supplies the address of four
// consecutive 16-bit elements X[k0 + r/4][n0 + 4*(r%4) ..] and lane i of the group receives
// X[k0 + 0..3][n0 + i].
template <typename E, int D>
struct OperandOffsets {
    typedef LdsTile<E, D> L;
    static constexpr int NJ = L::CH / 2;
    static constexpr int DB = (D + 31) / 32;
    static constexpr bool kHalfAffine = L::CH >= 16;  // +16 rows keeps the swizzle key (mod 16)
    static constexpr int NS_TR = kHalfAffine ? 1 : 2;
    static constexpr int ROW_BYTES = L::CH * 16;
    int row[NJ];
    int tr[Elem<E>::k16 ? DB : 1][NS_TR][2];

    __device__ __forceinline__ void init(int lane) {
        const int n = lane & 31, h = lane >> 5;
#pragma unroll
        for (int j = 0; j < NJ; j++) row[j] = L::chunk_off(n, 2 * j + h);
        if constexpr (Elem<E>::k16) {
            const int r = lane & 15, colgrp = (lane >> 4) & 1;
#pragma unroll
            for (int db = 0; db < DB; db++) {
                int col = 32 * db + 16 * colgrp + 4 * (r & 3);
                if (D < 32) col &= (D - 1);
#pragma unroll
                for (int s = 0; s < NS_TR; s++)
#pragma unroll
                    for (int w = 0; w < 2; w++) tr[db][s][w] = L::elem_off(16 * s + 8 * w + 4 * h + (r >> 2), col);
            }
        }
    }

    __device__ __forceinline__ i32x4 row_chunk(const lds_char* tile, int kb, int j, int lane) const {
        if constexpr (L::kBlockAffine) {
            return *reinterpret_cast<const lds_i32x4*>(tile + row[j] + kb * L::BLOCK_BYTES);
        } else {
            return *reinterpret_cast<const lds_i32x4*>(tile + L::chunk_off(32 * kb + (lane & 31), 2 * j + (lane >> 5)));
        }
    }

    // Transposed 16-bit operand: rows {32*kb + 16*s + 4*h + (0..3), + 8} at column 32*db + n.
    __device__ __forceinline__ i32x4 tr_operand(const lds_char* tile, int kb, int s, int db, int lane) const {
        const lds_char *a0, *a1;
        if constexpr (L::kBlockAffine) {
            const int imm = kb * L::BLOCK_BYTES + (kHalfAffine ? s * 16 * ROW_BYTES : 0);
            a0 = tile + tr[db][kHalfAffine ? 0 : s][0] + imm;
            a1 = tile + tr[db][kHalfAffine ? 0 : s][1] + imm;
        } else {
            const int r = lane & 15, colgrp = (lane >> 4) & 1, h = lane >> 5;
            int col = 32 * db + 16 * colgrp + 4 * (r & 3);
            if (D < 32) col &= (D - 1);
            const int rw = 32 * kb + 16 * s + 4 * h + (r >> 2);
            a0 = tile + L::elem_off(rw, col);
            a1 = tile + L::elem_off(rw + 8, col);
        }
        i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)a0);
        i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)a1);
        i16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(i32x4, v);
    }
};

// The same operands through per-lane POINTERS that already include everything wave-dependent (the
// LDS base, the wave's 32-row block of a tile, a region's place in LDS): what a use adds is a
// compile-time constant, which goes into the offset field of the LDS instruction, so a loop over tiles
// at fixed places spends no vector instruction on addresses.  The pointers pass through an empty asm:
// the compiler keeps them in registers instead of re-deriving them at every use.  Block-affine 16-bit
// tiles only; offsets must stay below 64 KiB.
template <typename E, int D>
struct OperandPointers {
    typedef LdsTile<E, D> L;
    typedef OperandOffsets<E, D> O;
    const lds_char* row[O::NJ];
    const lds_char* tr[O::DB][O::NS_TR][2];

    template <bool WITH_TR>
    __device__ __forceinline__ void init(const O& ofs, const lds_char* base) {
        static_assert(L::kBlockAffine && Elem<E>::k16, "block-affine 16-bit tiles");
#pragma unroll
        for (int j = 0; j < O::NJ; j++) {
            row[j] = base + ofs.row[j];
            asm volatile("" : "+v"(row[j]));
        }
        if constexpr (WITH_TR) {
#pragma unroll
            for (int db = 0; db < O::DB; db++)
#pragma unroll
                for (int s = 0; s < O::NS_TR; s++)
#pragma unroll
                    for (int w = 0; w < 2; w++) {
                        tr[db][s][w] = base + ofs.tr[db][s][w];
                        asm volatile("" : "+v"(tr[db][s][w]));
                    }
        }
    }
    // rows 0..31 of the tile `imm` bytes behind the base
    __device__ __forceinline__ i32x4 row_chunk(int imm, int j) const {
        return *reinterpret_cast<const lds_i32x4*>(row[j] + imm);
    }
    __device__ __forceinline__ i32x4 tr_operand(int imm, int s, int db) const {
        const int at = imm + (O::kHalfAffine ? s * 16 * O::ROW_BYTES : 0);
        i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(tr[db][O::kHalfAffine ? 0 : s][0] + at));
        i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(tr[db][O::kHalfAffine ? 0 : s][1] + at));
        i16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(i32x4, v);
    }
};

// acc(32 rows of the LDS tile x 32 cols) += X[32*kb + 0..31][:] * B^T, B = resident rows.
template <typename E, int D>
__device__ __forceinline__ f32x16 mma_rowwise(const lds_char* tile, int kb, const OperandOffsets<E, D>& ofs,
                                              const Resident<E, D>& b, f32x16 acc, int lane) {
#pragma unroll
    for (int j = 0; j < Resident<E, D>::NJ; j++) acc = Elem<E>::mma(ofs.row_chunk(tile, kb, j, lane), b.c[j], acc);
    return acc;
}

// The two 16-bit B operands a 32x32 accumulator-layout block packs into: operand s holds, for lane
// (n, h), rows {16*s + 8*(e/4) + 4*h + e%4, e = 0..7} of column n.
template <typename E>
__device__ __forceinline__ void pack_block(const f32x16& p, i32x4 (&bop)[2]) {
#pragma unroll
    for (int s = 0; s < 2; s++) {
        f32x8 ps;
#pragma unroll
        for (int e = 0; e < 8; e++) ps[e] = p[8 * s + e];
        bop[s] = Elem<E>::pack8(ps);
    }
}

// acc(32 out-rows x 32 cols) += X^T * P: contraction over the 32 rows of block kb of the LDS tile,
// P a 32x32 accumulator-layout block (rows = contraction index) reused as B operand, output row
// index = column 32*db + n of the LDS tile.  All DB head-dim blocks share the packed P operand.
template <typename E, int D>
__device__ __forceinline__ void mma_transposed(const lds_char* tile, int kb, const OperandOffsets<E, D>& ofs,
                                               const f32x16& p, f32x16 (&acc)[(D + 31) / 32], int lane) {
    constexpr int DB = (D + 31) / 32;
    if constexpr (Elem<E>::k16) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            f32x8 ps;
#pragma unroll
            for (int e = 0; e < 8; e++) ps[e] = p[8 * s + e];
            const i32x4 bop = Elem<E>::pack8(ps);
#pragma unroll
            for (int db = 0; db < DB; db++) acc[db] = Elem<E>::mma(ofs.tr_operand(tile, kb, s, db, lane), bop, acc[db]);
        }
    } else {
        typedef LdsTile<E, D> L;
        int h = lane >> 5;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int rw = 32 * kb + 8 * (r / 4) + 4 * h + (r % 4);
#pragma unroll
            for (int db = 0; db < DB; db++) {
                int col = 32 * db + (lane & 31);
                if (D < 32) col &= (D - 1);
                float a = *reinterpret_cast<const lds_float*>(tile + L::elem_off(rw, col));
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, p[r], acc[db], 0, 0, 0);
            }
        }
    }
}

// acc^T += X^T P with X the 32 rows behind the pointers (see OperandPointers)
template <typename E, int D>
__device__ __forceinline__ void mma_transposed(int imm, const OperandPointers<E, D>& ptrs, const f32x16& p,
                                               f32x16 (&acc)[(D + 31) / 32]) {
    constexpr int DB = (D + 31) / 32;
#pragma unroll
    for (int s = 0; s < 2; s++) {
        f32x8 ps;
#pragma unroll
        for (int e = 0; e < 8; e++) ps[e] = p[8 * s + e];
        const i32x4 bop = Elem<E>::pack8(ps);
#pragma unroll
        for (int db = 0; db < DB; db++) acc[db] = Elem<E>::mma(ptrs.tr_operand(imm, s, db), bop, acc[db]);
    }
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

// delta of the lane's row, sum over the head dim of O * dO (utils.py:94-217), for a dQ kernel that keeps
// the row's dO chunks as a resident operand: the same chunks of O are read here, every lane sums its
// half of the row and the row's two lanes add up.  Rows >= rows_valid give 0.  All 64 lanes must call.
template <typename E, int D>
__device__ __forceinline__ float resident_row_delta(const Resident<E, D>& dof, const typename Elem<E>::type* o_rows,
                                                    int64_t o_stride, int rows_valid, int lane) {
    using ET = typename Elem<E>::type;
    constexpr int NJ = Resident<E, D>::NJ;
    constexpr int EPC = 16 / Elem<E>::kBytes;
    Resident<E, D> of;
    load_resident<E, D>(of, o_rows, o_stride, rows_valid, lane);
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        // (plain conversions and fused multiply-adds: v_dot2_f32_bf16 gave wrong sums here)
        const ET* a = reinterpret_cast<const ET*>(&of.c[j]);
        const ET* d = reinterpret_cast<const ET*>(&dof.c[j]);
#pragma unroll
        for (int e = 0; e < EPC; e++) acc += Elem<E>::to_float(a[e]) * Elem<E>::to_float(d[e]);
    }
    return acc + __shfl_xor(acc, 32, 64);
}

// Store one output row from transposed accumulators: lane (n, h) holds, for every 32-wide block
// db of the head dim, the 16 values of columns d = 32*db + 8*(r/4) + 4*h + r%4 of ITS row.
// Each group of four consecutive r is four consecutive d.  fp32: one 16-byte store per group.  16-bit
// types: the two lanes of a row trade one 8-byte group of every pair (v_permlane32_swap), so that each
// writes 16 contiguous bytes and a store instruction covers 32 contiguous bytes of every row (8-byte
// stores scattered over 32 rows reach HBM as partial sectors: the forward wrote 1.33x its output).
// Both lanes of a row must be active or inactive together.  Rows that are not `valid` are written as zeros.
template <typename E, int D>
__device__ __forceinline__ void store_row_transposed(typename Elem<E>::type* row_ptr,
                                                     const f32x16 (&acc)[(D + 31) / 32], float mult,
                                                     bool valid, int h) {
    constexpr int DB = (D + 31) / 32;
#pragma unroll
    for (int db = 0; db < DB; db++) {
        if constexpr (Elem<E>::k16) {
#pragma unroll
            for (int gp = 0; gp < 2; gp++) {
                if (D >= 32 || 16 * gp < D) {
                    f32x4 va, vb;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        va[e] = valid ? acc[db][8 * gp + e] * mult : 0.f;
                        vb[e] = valid ? acc[db][8 * gp + 4 + e] * mult : 0.f;
                    }
                    const i32x2 a = Elem<E>::pack4(va), b = Elem<E>::pack4(vb);
                    // first: lanes h = 0 keep their group 2 gp, lanes h = 1 receive the partner's group 2 gp + 1;
                    // second: lanes h = 0 receive the partner's group 2 gp, lanes h = 1 keep their group 2 gp + 1
                    const auto w0 = __builtin_amdgcn_permlane32_swap(a[0], b[0], false, false);
                    const auto w1 = __builtin_amdgcn_permlane32_swap(a[1], b[1], false, false);
                    *reinterpret_cast<i32x4*>(row_ptr + 32 * db + 16 * gp + 8 * h) =
                        i32x4{(int)w0[0], (int)w1[0], (int)w0[1], (int)w1[1]};
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                int d0 = 32 * db + 8 * g + 4 * h;
                if (D >= 32 || d0 < D) {
                    f32x4 vals;
#pragma unroll
                    for (int e = 0; e < 4; e++) vals[e] = valid ? acc[db][4 * g + e] * mult : 0.f;
                    *reinterpret_cast<f32x4*>(row_ptr + d0) = vals;
                }
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

// (work-item order: xcd_contiguous_item, chill_tiles.h)

}  // namespace chill
