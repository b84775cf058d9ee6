// Pieces of the logical -> physical redirect shared by the kernels that run it
// (map.hip: the streaming redirect; plan.hip: the one-launch plan).
#pragma once
#include "common.h"

namespace lplb {

// Per-expert constants of the redirect, one 16-byte LDS read per token.
struct __attribute__((aligned(16))) ExpertEntry {
  int32_t total;     // tokens of this expert in the whole index array
  uint32_t magic;    // floor((2^32 - 1) / total), 0 for total <= 0
  int32_t expected;  // tokens that stay on the original, trunc(o_weight * total)
  int32_t original;  // physical slot of the original
};

// State of one expert inside one wave, one 16-byte LDS read / write per token.
struct __attribute__((aligned(16))) WaveSlot {
  int32_t next;             // ordinal of the wave's next token of this expert
  int32_t unused;
  unsigned long long bits;  // lanes of the current chunk that hold this expert
};

// h mod total with C's truncating sign rule.  magic = floor((2^32 - 1) / total) is at
// least 2^32 / total - 1, so for a <= 2^31: a / total >= a * magic / 2^32 >=
// a / total - 1/2.  q = mulhi(a, magic) is therefore the true quotient or one less,
// and one conditional subtract finishes (a 32-bit division per expert instead of one
// per token).
// WRAP: the hash 499 k + 41 may have wrapped to negative.
template <bool WRAP> __device__ inline int32_t hashed_mod(int32_t h, const ExpertEntry &x) {
  const uint32_t a = WRAP ? (uint32_t)max(h, -h) : (uint32_t)h;
  uint32_t r = a - __umulhi(a, x.magic) * (uint32_t)x.total;
  r = min(r, r - (uint32_t)x.total);           // one conditional subtract
  int32_t m = (WRAP && h < 0) ? -(int32_t)r : (int32_t)r;
  return x.total > 0 ? m : 0;
}

constexpr int kMaxWaves = 16;
typedef int i32x4 __attribute__((ext_vector_type(4)));


// The shapes the table build needs.
struct RedirectShape {
  int n_logical, n_ranks, G, D, C, L, P;
};

// table / replica / first ordinal of expert e: total tokens t, of which `start` lie
// before this workgroup's slice.  minilp.cu:466-496.
__device__ inline void init_entry(ExpertEntry *table, int32_t *replica, int32_t *carry, int e, int32_t t,
                                  int32_t start) {
  ExpertEntry x;
  x.total = t;
  x.magic = t >= 1 ? 0xffffffffu / (uint32_t)t : 0u;
  x.expected = t;
  x.original = -1;
  table[e] = x;
  replica[e] = -1;
  carry[e] = start;
}
// Physical slot e holds logical expert le as its original.
__device__ inline void set_original(ExpertEntry *table, const RedirectShape &sh, int e, int le) {
  if (le >= 0 && le < sh.n_logical)
    table[le].original = (e / sh.L) * sh.P + (e % sh.L);
}
// Replica slot `local` of EP rank ep_rank copies logical expert le; the copy lives on
// group rank `host`.
__device__ inline void set_replica_slot(int32_t *replica, const RedirectShape &sh, int ep_rank, int local, int le,
                                        int host) {
  if (le >= 0 && le < sh.n_logical)
    replica[le] = ((ep_rank / sh.G) * sh.G + host + 1) * sh.P - sh.C * sh.D + local;
}
// Tokens of an expert with `total` tokens that stay on its original when the original
// keeps `share` of them: the fp32 product truncated toward zero (saturating, NaN -> 0).
__device__ inline int32_t expected_on_original(float share, int32_t total) {
  return __float2int_rz(share * (float)total);
}
// Both at once.
__device__ inline void set_replica(ExpertEntry *table, int32_t *replica, const RedirectShape &sh, int ep_rank,
                                   int local, int le, float share, int host) {
  if (le >= 0 && le < sh.n_logical)
    table[le].expected = expected_on_original(share, table[le].total);
  set_replica_slot(replica, sh, ep_rank, local, le, host);
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

// Tokens per physical expert, = bincount of the redirect's output, from the tables
// of any one workgroup: every slot is the original or the replica of its logical expert.
__device__ inline void emit_physical_counts(const ExpertEntry *table, const int32_t *replica,
                                            const RedirectShape &sh, const int32_t *phy2log, int32_t *counts,
                                            int tid, int nt) {
  for (int i = tid; i < sh.n_ranks * sh.P; i += nt) {
    const int le = phy2log[i];
    int32_t v = 0;
    if (le >= 0 && le < sh.n_logical) {
      const ExpertEntry x = table[le];
      const int32_t kept = kept_on_original(x.total, x.expected);
      if (x.original == i)
        v = kept;
      else if (replica[le] == i)
        v = x.total - kept;
    }
    counts[i] = v;
  }
}

// One token of a 64-index chunk: lanes holding the same expert find each other
// through the wave's 64-bit bitmap for that expert; the rank among those peers is a
// popcount of lower lanes and the last peer advances the wave's ordinal.  Returns
// the token's hash (499 k + 41) mod total (minilp.cu:505) and, in x, its expert's
// entry; neither is defined for e < 0.  All lanes of the wave call it together and
// put a wave barrier between chunks.  It does not read x.expected, so it may run
// before the LP's shares are known.
template <bool WRAP>
__device__ inline int32_t hash_of_token(int e, WaveSlot *mine, const ExpertEntry *table, unsigned long long my_bit,
                                        ExpertEntry &x) {
  const bool valid = e >= 0;
  if (valid)
    atomicOr(&mine[e].bits, my_bit);
  int32_t h = 0;
  if (valid) {
    const i32x4 sraw = *reinterpret_cast<const i32x4 *>(&mine[e]);
    const i32x4 xraw = *reinterpret_cast<const i32x4 *>(&table[e]);
    const uint32_t peers_lo = (uint32_t)sraw.z, peers_hi = (uint32_t)sraw.w;
    const int rank = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
    const int cnt = __popc(peers_lo) + __popc(peers_hi);
    const int32_t k = sraw.x + rank;
    x.total = xraw.x; x.magic = (uint32_t)xraw.y; x.expected = xraw.z; x.original = xraw.w;
    h = hashed_mod<WRAP>((int32_t)((uint32_t)k * 499u + 41u), x);
    if (rank == cnt - 1)   // last peer: advance the ordinal, clear the bitmap
      *reinterpret_cast<i32x4 *>(&mine[e]) = i32x4{k + 1, 0, 0, 0};
  }
  return h;
}

// The physical expert of a token of expert e with hash h (-1 for e < 0).
template <bool WRAP>
__device__ inline int64_t redirect_token(int e, WaveSlot *mine, const ExpertEntry *table, const int32_t *replica,
                                         unsigned long long my_bit) {
  ExpertEntry x;
  const int32_t h = hash_of_token<WRAP>(e, mine, table, my_bit, x);
  int64_t o = -1;
  if (e >= 0)
    o = h >= x.expected ? replica[e] : x.original;
  return o;
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
    ExpertEntry x;
    x.total = total;
    x.magic = magic;
    return hashed_mod<true>((int32_t)((uint32_t)k * 499u + 41u), x);
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
