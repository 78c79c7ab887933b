// How to write a mask functor for a user-mask build (make USER_MASK=<file> BUILD=<dir> LIBDIR=<dir>).
//
// This file is documentation plus a worked example; it is what `make USER_MASK=chill_user_mask.h`
// compiles.  The counterpart in the reference is a ChillMask subclass whose Triton static methods
// are compiled on first use ("Creating Your Own Mask", README.md:124-179; contract mask.py:54-250).
//
// The file is included at namespace scope after chill_mask.h's own definitions and must specialise
// chill::Mask<CHILL_MASK_USER>, deriving from MaskDefaults.  Required members:
//
//   static constexpr int kNumArgs            number of integer arguments (0..4), read as a.a0 .. a.a3
//   pred(q, k, seq_len, a)                   true if query q may attend to key k   (mask.py:54-77)
//   k_range_for_q(q, seq_len, a)             INCLUSIVE {lo, hi} of the keys q can see (mask.py:93-107)
//   q_range_for_k(k, seq_len, a)             INCLUSIVE {lo, hi} of the queries that see k (mask.py:79-91)
//
// Optional members (defaults in MaskDefaults = the reference's base class):
//
//   kMonotoneLimits = false                  if lo or hi of a range ever DEcreases from one position to
//                                            the next; tile ranges are then the hull over a tile's rows
//   kHasKFullRange / k_full_range_for_q      HALF-OPEN key range every query of a tile sees entirely
//   kHasQFullRange / q_full_range_for_k      same for a key tile                    (mask.py:110-151)
//   has_full_blocks / is_full_block          blocks that need no predicate          (mask.py:212-250)
//   kSafe                                    every query sees at least one key
//
// Every function is CHILL_HD static, takes positions as non-negative ints and the arguments as
// MaskArgs; the range rules must return the exact minimum and maximum (ChillMask.verify checks it).
//
// Example: "attention sinks + causal window" — a query sees the first a0 keys and the a1 keys before it.
#pragma once

namespace chill {

template <>
struct Mask<CHILL_MASK_USER> : MaskDefaults {
    static constexpr int kNumArgs = 2;            // a0 = number of sink keys, a1 = window
    static constexpr bool kSafe = true;           // a query always sees itself
    static constexpr bool kMonotoneLimits = false;  // q_range_for_k's upper limit drops after the sinks
    CHILL_HD static bool pred(int q, int k, int, MaskArgs a) {
        return (k <= q) && ((k < a.a0) || (q - k <= a.a1));
    }
    CHILL_HD static Range k_range_for_q(int q, int, MaskArgs a) {
        return {a.a0 > 0 ? 0 : imax(0, q - a.a1), q};
    }
    CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs a) {
        return {k, k < a.a0 ? seq_len - 1 : imin(k + a.a1, seq_len - 1)};
    }
};

}  // namespace chill
