// Pieces of the logical -> physical redirect shared by the kernels that run it
// (map.hip: the streaming redirect; plan.hip: the one-launch plan).
#pragma once
#include "common.h"

namespace lplb {

// h mod total with C's truncating sign rule.  magic = floor((2^32 - 1) / total) is at
// least 2^32 / total - 1, so for a <= 2^31: a / total >= a * magic / 2^32 >=
// a / total - 1/2.  q = mulhi(a, magic) is therefore the true quotient or one less,
// and one conditional subtract finishes (a 32-bit division per expert instead of one
// per token).
// WRAP: the hash 499 k + 41 may have wrapped to negative.
template <bool WRAP> __device__ inline int32_t hashed_mod(int32_t h, int32_t total, uint32_t magic) {
  const uint32_t a = WRAP ? (uint32_t)max(h, -h) : (uint32_t)h;
  uint32_t r = a - __umulhi(a, magic) * (uint32_t)total;
  r = min(r, r - (uint32_t)total);           // one conditional subtract
  int32_t m = (WRAP && h < 0) ? -(int32_t)r : (int32_t)r;
  return total > 0 ? m : 0;
}

constexpr int kMaxWaves = 16;
typedef int i32x4 __attribute__((ext_vector_type(4)));

// The shapes the table build needs.
struct RedirectShape {
  int n_logical, n_ranks, G, D, C, L, P;
};

// Tokens of an expert with `total` tokens that stay on the original when the original
// keeps `share` of them: the fp32 product truncated toward zero (saturating, NaN -> 0).
__device__ inline int32_t expected_on_original(float share, int32_t total) {
  return __float2int_rz(share * (float)total);
}

// How many of an expert's `total` tokens stay on the original:
// #{k in [0, total) : (499 k + 41) mod total < expected}.  499 is prime, so unless it
// divides total the hash is a bijection on [0, total) and the answer is expected
// clamped to [0, total]; if total = 499 m the hash is 499 (k mod m) + 41, each value
// taken 499 times.  Valid while 499 k + 41 stays below 2^31.
__device__ inline int32_t kept_on_original(int32_t total, int32_t expected) {
  if (total <= 0)
    return 0;
  const int32_t want = min(max(expected, 0), total);
  if (total % 499 != 0)
    return want;
  const int32_t m = total / 499;
  return 499 * (want > 41 ? min(m, (want - 41 + 498) / 499) : 0);
}

// ---------------------------------------------------------------------------
// Redirect with ordinals only where they matter.
//
// The ordinal k of a token decides between original and replica, so only tokens of
// experts that HAVE a replica need one: every other expert's tokens go to its
// original slot whatever k is (expected == total, minilp.cu:466-470).  The tables
// are therefore split: a route per logical expert (original slot + index of its
// replicated set, if any) and, per replicated set, the constants of the hash test.
// Ranking state exists per replicated set only, which is what keeps it small.

// Per logical expert; entry n_logical is the route of masked / out-of-range tokens.
struct __attribute__((aligned(8))) Route {
  int32_t original;  // physical slot of the original, -1 if none
  int32_t rep;       // index of the replicated set this expert belongs to; n_rep if it has no replica
};
// Per replicated set (ep_rank, slot) in the order of minilp.cu:478-495; entry n_rep is a
// stand-in for "no replica" whose test never sends a token away (expected = INT32_MAX).
struct __attribute__((aligned(16))) RepEntry {
  int32_t total;     // tokens of the expert in the whole index array
  uint32_t magic;    // floor((2^32 - 1) / total), 0 for total <= 0
  int32_t expected;  // tokens that stay on the original, trunc(o_weight * total)
  int32_t replica;   // physical slot of the replica
};
// One 64-index chunk of one wave and one replicated set.
struct __attribute__((aligned(16))) ChunkSlot {
  uint32_t bits_lo, bits_hi;  // lanes of the chunk that hold a token of the set
  int32_t start;              // ordinal of the first of them
  int32_t unused;
};

// Bytes of the ranking record of one (wave, replicated set): K chunk slots for each of
// the two pass parities, padded to an odd multiple of 16 bytes so that consecutive
// sets start in different LDS banks.
constexpr int rank_record_bytes(int k) { return 2 * k * (int)sizeof(ChunkSlot) + 16; }

// (499 k + 41) mod total with the sign rule of C (minilp.cu:505), k >= 0.
// !WRAP: k < 2^24 and 499 k + 41 < 2^31 (the caller guarantees it).
template <bool WRAP> __device__ inline int32_t ordinal_hash(int32_t k, int32_t total, uint32_t magic) {
  if constexpr (WRAP) {
    return hashed_mod<true>((int32_t)((uint32_t)k * 499u + 41u), total, magic);
  } else {
    const uint32_t a = __umul24((uint32_t)k, 499u) + 41u;
    const uint32_t r = a - __umulhi(a, magic) * (uint32_t)total;   // true remainder, or that plus total
    return (int32_t)min(r, r - (uint32_t)total);
  }
}

// Exact n / d for n < 65536 and 1 <= d < 65536 with m = fast_div_magic(d) =
// floor(2^32 / d) + 1: m d = 2^32 + delta with 0 < delta <= d, so n m / 2^32 exceeds
// n / d by n delta / (d 2^32) < 1 / d, too little to reach the next integer.  d = 1
// (m would be 2^32 + 1) is encoded as m = 0.
__host__ __device__ inline uint32_t fast_div_magic(uint32_t d) {
  return d <= 1 ? 0u : (uint32_t)(0x100000000ull / d) + 1u;
}
__device__ inline uint32_t fast_div(uint32_t n, uint32_t m) { return m ? __umulhi(n, m) : n; }

// DPP row shift right by N lanes inside a row of 16 (lanes without a source get 0).
template <int N> __device__ inline int row_shr(int v) {
  return __builtin_amdgcn_update_dpp(0, v, 0x110 + N, 0xF, 0xF, true);
}
template <int CTRL> __device__ inline int dpp_int(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
// Sum over each group of K adjacent lanes (K = 1, 2, 4, 8 or 16; every lane gets its group's sum).
template <int K> __device__ inline int group_sum(int v) {
  if constexpr (K >= 2) v += dpp_int<0xB1>(v);    // quad_perm [1,0,3,2]
  if constexpr (K >= 4) v += dpp_int<0x4E>(v);    // quad_perm [2,3,0,1]
  if constexpr (K >= 8) v += dpp_int<0x141>(v);   // row_half_mirror
  if constexpr (K >= 16) v += dpp_int<0x140>(v);  // row_mirror
  return v;
}
// Sum of the lanes before this one in its group of K adjacent lanes (pos = lane % K):
// an inclusive scan in log2(K) shift-and-add steps, minus the lane's own value.
template <int K> __device__ inline int group_exclusive_scan(int v, int pos) {
  int acc = v;
  if constexpr (K >= 2) { const int t = row_shr<1>(acc); acc += pos >= 1 ? t : 0; }
  if constexpr (K >= 4) { const int t = row_shr<2>(acc); acc += pos >= 2 ? t : 0; }
  if constexpr (K >= 8) { const int t = row_shr<4>(acc); acc += pos >= 4 ? t : 0; }
  if constexpr (K >= 16) { const int t = row_shr<8>(acc); acc += pos >= 8 ? t : 0; }
  return acc - v;
}

// Ranking record of one (wave, replicated set) when a slice is a single pass: K chunk
// slots; from four slots on padded to an odd multiple of 16 bytes (a record of 64, 128 or
// 256 bytes would put every set into the same LDS banks).
constexpr int rank_record_bytes_single(int k) { return k * (int)sizeof(ChunkSlot) + (k >= 4 ? 16 : 0); }

} // namespace lplb
