// Device bodies of the nonce-search kernels: SHA-256d, BLAKE2b-256 (Sia and
// ccminer header layouts) and Ethash.  The original kernels read their header,
// midstate, target and DAG pointer from __constant__ symbols written by their
// host program; here the launcher places the same values behind the original
// argument list in the kernel-argument segment, where gfx950 reads them with
// scalar loads into SGPRs.
#pragma once
#include <hip/hip_runtime.h>

#include "../../../include/hfuse_gfx950.h"
#include "subblock.h"

namespace hfuse {

typedef unsigned long long u64;
typedef unsigned int u32;

__device__ __forceinline__ u32 ror32(u32 x, int n) { return __builtin_rotateright32(x, n); }
// 64-bit rotates by a compile-time amount as two 32-bit funnel shifts
// (v_alignbit_b32); a rotate by 32 is a register swap.
__device__ __forceinline__ u64 ror64(u64 x, int n) {
  const u32 lo = (u32)x, hi = (u32)(x >> 32);
  u32 nlo, nhi;
  if (n == 0) return x;
  if (n == 32) { nlo = hi; nhi = lo; }
  else if (n < 32) { nlo = __builtin_amdgcn_alignbit(hi, lo, n); nhi = __builtin_amdgcn_alignbit(lo, hi, n); }
  else { nlo = __builtin_amdgcn_alignbit(lo, hi, n - 32); nhi = __builtin_amdgcn_alignbit(hi, lo, n - 32); }
  return ((u64)nhi << 32) | nlo;
}
__device__ __forceinline__ u64 rol64(u64 x, int n) { return ror64(x, (64 - n) & 63); }
__device__ __forceinline__ u32 bswap32(u32 x) { return __builtin_bswap32(x); }
__device__ __forceinline__ u64 bswap64(u64 x) { return __builtin_bswap64(x); }

// Appends one hit; slots beyond HF_MAX_SEARCH_RESULTS are counted but not stored.
struct Words8 {
  u32 w[8];
};
__device__ __noinline__ void record_hit(hf_search_results *out, u64 nonce, Words8 digest, Words8 mix) {
  const u32 slot = atomicAdd(&out->count, 1u);
  if (slot < HF_MAX_SEARCH_RESULTS) {
    hf_search_hit *h = &out->hit[slot];
    h->nonce = nonce;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      h->digest[i] = digest.w[i];
      h->mix[i] = mix.w[i];
    }
  }
}

// ----------------------------------------------------------------------------
// SHA-256d  (sha256d_gpu_hash_shared: scripts/data/ethminer_event.csv:26)
// ----------------------------------------------------------------------------
struct Sha256dDevArgs {
  u32 threads, start_nonce;
  hf_search_results *out;
  u32 midstate[8];  // state after the first 64 header bytes
  u32 tail[3];      // header bytes 64..75 as big-endian words
  u32 pad;
  u64 target64;     // top 64 bits of the little-endian 256-bit target
};

__device__ __constant__ const u32 kShaK[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
    0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
    0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
    0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
    0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
    0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
    0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
    0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

// One compression with a rolling 16-word schedule, fully unrolled so the round
// constants become instruction literals and constant message words fold away.
__device__ __forceinline__ void sha256_compress(u32 st[8], u32 w[16]) {
  u32 a = st[0], b = st[1], c = st[2], d = st[3], e = st[4], f = st[5], g = st[6], h = st[7];
#pragma unroll
  for (int i = 0; i < 64; i++) {
    if (i >= 16) {
      const u32 w15 = w[(i - 15) & 15], w2 = w[(i - 2) & 15];
      const u32 s0 = ror32(w15, 7) ^ ror32(w15, 18) ^ (w15 >> 3);
      const u32 s1 = ror32(w2, 17) ^ ror32(w2, 19) ^ (w2 >> 10);
      w[i & 15] = w[i & 15] + s0 + w[(i - 7) & 15] + s1;
    }
    const u32 S1 = ror32(e, 6) ^ ror32(e, 11) ^ ror32(e, 25);
    const u32 ch = (e & f) ^ (~e & g);
    const u32 t1 = h + S1 + ch + kShaK[i] + w[i & 15];
    const u32 S0 = ror32(a, 2) ^ ror32(a, 13) ^ ror32(a, 22);
    const u32 mj = (a & b) ^ (a & c) ^ (b & c);
    h = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + S0 + mj;
  }
  st[0] += a; st[1] += b; st[2] += c; st[3] += d; st[4] += e; st[5] += f; st[6] += g; st[7] += h;
}

struct Sha256dBody {
  static constexpr KernelId kId = K_SHA256D;
  using Args = Sha256dDevArgs;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned) {
    // 64-bit counter: `threads` may be anything up to 2^32 - 1, so t + stride must not wrap
    const u64 stride = sb.gstride();
    for (u64 t = sb.gtid(); t < a.threads; t += stride) {
      const u32 nonce = a.start_nonce + (u32)t;
      u32 st[8], w[16];
#pragma unroll
      for (int i = 0; i < 8; i++) st[i] = a.midstate[i];
      w[0] = a.tail[0]; w[1] = a.tail[1]; w[2] = a.tail[2];
      w[3] = bswap32(nonce);  // header bytes 76..79 hold the nonce little-endian
      w[4] = 0x80000000u;
#pragma unroll
      for (int i = 5; i < 15; i++) w[i] = 0;
      w[15] = 640;
      sha256_compress(st, w);
#pragma unroll
      for (int i = 0; i < 8; i++) w[i] = st[i];
      w[8] = 0x80000000u;
#pragma unroll
      for (int i = 9; i < 15; i++) w[i] = 0;
      w[15] = 256;
      st[0] = 0x6a09e667; st[1] = 0xbb67ae85; st[2] = 0x3c6ef372; st[3] = 0xa54ff53a;
      st[4] = 0x510e527f; st[5] = 0x9b05688c; st[6] = 0x1f83d9ab; st[7] = 0x5be0cd19;
      sha256_compress(st, w);
      // digest bytes 24..31 read little-endian = top 64 bits of the 256-bit value
      const u64 top = ((u64)bswap32(st[7]) << 32) | bswap32(st[6]);
      if (top <= a.target64) {
        Words8 dg, zero = {};
#pragma unroll
        for (int i = 0; i < 8; i++) dg.w[i] = bswap32(st[i]);
        record_hit(a.out, nonce, dg, zero);
      }
    }
  }
};

// ----------------------------------------------------------------------------
// BLAKE2b-256 of an 80-byte header
// (sia_blake2b_gpu_hash / blake2b_gpu_hash: scripts/data/ethminer_event.csv:2,22)
// ----------------------------------------------------------------------------
struct Blake2bDevArgs {
  u32 threads, start_nonce;
  hf_search_results *out;
  u64 target64;  // hit iff the first 8 digest bytes, read big-endian, are <= target64
  u64 m[10];     // the header as ten little-endian words
};

__device__ __constant__ const u64 kB2IV[8] = {0x6a09e667f3bcc908ull, 0xbb67ae8584caa73bull, 0x3c6ef372fe94f82bull,
                                              0xa54ff53a5f1d36f1ull, 0x510e527fade682d1ull, 0x9b05688c2b3e6c1full,
                                              0x1f83d9abfb41bd6bull, 0x5be0cd19137e2179ull};

__device__ __constant__ const unsigned char kB2Sigma[12][16] = {
    {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3},
    {11, 8, 12, 0, 5, 2, 15, 13, 10, 14, 3, 6, 7, 1, 9, 4}, {7, 9, 3, 1, 13, 12, 11, 14, 2, 6, 5, 10, 4, 0, 15, 8},
    {9, 0, 5, 7, 2, 4, 10, 15, 14, 1, 11, 12, 6, 8, 3, 13}, {2, 12, 6, 10, 0, 11, 8, 3, 4, 13, 7, 5, 15, 14, 1, 9},
    {12, 5, 1, 15, 14, 13, 4, 10, 0, 7, 6, 3, 9, 2, 8, 11}, {13, 11, 7, 14, 12, 1, 3, 9, 5, 0, 15, 4, 8, 6, 2, 10},
    {6, 15, 14, 9, 11, 3, 0, 8, 12, 2, 13, 7, 1, 4, 10, 5}, {10, 2, 8, 4, 7, 6, 1, 5, 15, 11, 9, 14, 3, 12, 13, 0},
    {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3}};

#define HF_B2_G(a, b, c, d, x, y) \
  do {                            \
    a = a + b + (x);              \
    d = ror64(d ^ a, 32);         \
    c = c + d;                    \
    b = ror64(b ^ c, 24);         \
    a = a + b + (y);              \
    d = ror64(d ^ a, 16);         \
    c = c + d;                    \
    b = ror64(b ^ c, 63);         \
  } while (0)

// Twelve rounds over an 80-byte single final block; m[10..15] are zero.
__device__ __forceinline__ void blake2b_80_rounds(u64 v[16], const u64 m[16]) {
#pragma unroll
  for (int r = 0; r < 12; r++) {
    const unsigned char *s = kB2Sigma[r];
    HF_B2_G(v[0], v[4], v[8], v[12], m[s[0]], m[s[1]]);
    HF_B2_G(v[1], v[5], v[9], v[13], m[s[2]], m[s[3]]);
    HF_B2_G(v[2], v[6], v[10], v[14], m[s[4]], m[s[5]]);
    HF_B2_G(v[3], v[7], v[11], v[15], m[s[6]], m[s[7]]);
    HF_B2_G(v[0], v[5], v[10], v[15], m[s[8]], m[s[9]]);
    HF_B2_G(v[1], v[6], v[11], v[12], m[s[10]], m[s[11]]);
    HF_B2_G(v[2], v[7], v[8], v[13], m[s[12]], m[s[13]]);
    HF_B2_G(v[3], v[4], v[9], v[14], m[s[14]], m[s[15]]);
  }
}

__device__ __forceinline__ void blake2b_80_init(u64 v[16]) {
#pragma unroll
  for (int i = 0; i < 8; i++) { v[i] = kB2IV[i]; v[i + 8] = kB2IV[i]; }
  v[0] ^= 0x01010020ull;  // digest length 32, fanout 1, depth 1
  v[12] ^= 80;            // byte counter
  v[14] = ~v[14];         // final block
}

// The rare path: recompute the whole digest for a nonce that passed the test.
template <int NONCE_WORD, bool NONCE_HIGH>
__device__ __forceinline__ void blake2b_record(const Blake2bDevArgs &a, u32 nonce) {
  u64 m[16], v[16];
#pragma unroll
  for (int i = 0; i < 10; i++) m[i] = a.m[i];
#pragma unroll
  for (int i = 10; i < 16; i++) m[i] = 0;
  if (NONCE_HIGH) m[NONCE_WORD] = (m[NONCE_WORD] & 0xFFFFFFFFull) | ((u64)nonce << 32);
  else m[NONCE_WORD] = (m[NONCE_WORD] & 0xFFFFFFFF00000000ull) | nonce;
  blake2b_80_init(v);
  blake2b_80_rounds(v, m);
  Words8 dg, zero = {};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    u64 h = kB2IV[i] ^ v[i] ^ v[i + 8];
    if (i == 0) h ^= 0x01010020ull;
    dg.w[2 * i] = (u32)h;
    dg.w[2 * i + 1] = (u32)(h >> 32);
  }
  record_hit(a.out, NONCE_HIGH ? (u64)nonce : m[NONCE_WORD], dg, zero);
}

// NONCE_WORD/NONCE_HIGH: Sia puts the running 32-bit nonce in the low half of
// word 4 (byte 32); ccminer's layout in the high half of word 9 (byte 76).
template <int NONCE_WORD, bool NONCE_HIGH>
struct Blake2bBody {
  static constexpr KernelId kId = NONCE_HIGH ? K_BLAKE2B : K_SIA_BLAKE2B;
  using Args = Blake2bDevArgs;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = true;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned) {
    const u64 stride = sb.gstride();  // 64-bit counter: t + stride must not wrap for any `threads`
    for (u64 t = sb.gtid(); t < a.threads; t += stride) {
      const u32 nonce = a.start_nonce + (u32)t;
      u64 m[16], v[16];
#pragma unroll
      for (int i = 0; i < 10; i++) m[i] = a.m[i];
#pragma unroll
      for (int i = 10; i < 16; i++) m[i] = 0;
      if (NONCE_HIGH) m[NONCE_WORD] = (m[NONCE_WORD] & 0xFFFFFFFFull) | ((u64)nonce << 32);
      else m[NONCE_WORD] = (m[NONCE_WORD] & 0xFFFFFFFF00000000ull) | nonce;
      blake2b_80_init(v);
      blake2b_80_rounds(v, m);
      const u64 h0 = kB2IV[0] ^ 0x01010020ull ^ v[0] ^ v[8];
      if (bswap64(h0) <= a.target64) blake2b_record<NONCE_WORD, NONCE_HIGH>(a, nonce);
    }
  }
};
using SiaBlake2bBody = Blake2bBody<4, false>;
using CcminerBlake2bBody = Blake2bBody<9, true>;

// ----------------------------------------------------------------------------
// Keccak-f[1600] and Ethash  (ethash_search: scripts/data/ethminer_event.csv:9)
// ----------------------------------------------------------------------------
__device__ __constant__ const u64 kKeccakRC[24] = {
    0x0000000000000001ull, 0x0000000000008082ull, 0x800000000000808aull, 0x8000000080008000ull,
    0x000000000000808bull, 0x0000000080000001ull, 0x8000000080008081ull, 0x8000000000008009ull,
    0x000000000000008aull, 0x0000000000000088ull, 0x0000000080008009ull, 0x000000008000000aull,
    0x000000008000808bull, 0x800000000000008bull, 0x8000000000008089ull, 0x8000000000008003ull,
    0x8000000000008002ull, 0x8000000000000080ull, 0x000000000000800aull, 0x800000008000000aull,
    0x8000000080008081ull, 0x8000000000008080ull, 0x0000000080000001ull, 0x8000000080008008ull};

// 24 rounds kept as a loop (one round is ~350 instructions; unrolling two
// permutations per hash would not fit the instruction cache).
__device__ __forceinline__ void keccak_f1600(u64 s[25]) {
#pragma unroll 1
  for (int round = 0; round < 24; round++) {
    u64 c[5], d;
#pragma unroll
    for (int x = 0; x < 5; x++) c[x] = s[x] ^ s[x + 5] ^ s[x + 10] ^ s[x + 15] ^ s[x + 20];
#pragma unroll
    for (int x = 0; x < 5; x++) {
      d = c[(x + 4) % 5] ^ rol64(c[(x + 1) % 5], 1);
#pragma unroll
      for (int y = 0; y < 25; y += 5) s[x + y] ^= d;
    }
    // rho + pi along the single 24-cycle of the lane permutation
    u64 t = s[1], u;
#define HF_RP(dst, r) u = s[dst]; s[dst] = rol64(t, r); t = u;
    HF_RP(10, 1)  HF_RP(7, 3)   HF_RP(11, 6)  HF_RP(17, 10) HF_RP(18, 15) HF_RP(3, 21)
    HF_RP(5, 28)  HF_RP(16, 36) HF_RP(8, 45)  HF_RP(21, 55) HF_RP(24, 2)  HF_RP(4, 14)
    HF_RP(15, 27) HF_RP(23, 41) HF_RP(19, 56) HF_RP(13, 8)  HF_RP(12, 25) HF_RP(2, 43)
    HF_RP(20, 62) HF_RP(14, 18) HF_RP(22, 39) HF_RP(9, 61)  HF_RP(6, 20)  HF_RP(1, 44)
#undef HF_RP
#pragma unroll
    for (int y = 0; y < 25; y += 5) {
      const u64 a0 = s[y], a1 = s[y + 1], a2 = s[y + 2], a3 = s[y + 3], a4 = s[y + 4];
      s[y] = a0 ^ (~a1 & a2);
      s[y + 1] = a1 ^ (~a2 & a3);
      s[y + 2] = a2 ^ (~a3 & a4);
      s[y + 3] = a3 ^ (~a4 & a0);
      s[y + 4] = a4 ^ (~a0 & a1);
    }
    s[0] ^= kKeccakRC[round];
  }
}

struct EthashDevArgs {
  hf_search_results *out;
  u64 start_nonce;
  const u32x4 *dag;  // n_items x 128 bytes
  u32 n_items;
  u32 pow2_mask;     // n_items - 1 when n_items is a power of two, else 0
  u64 target;        // hit iff the first 8 bytes of the final hash, big-endian, are <= target
  u64 header[4];
};

constexpr u32 kFnvPrime = 0x01000193u;
__device__ __forceinline__ u32 fnv(u32 a, u32 b) { return (a * kFnvPrime) ^ b; }
__device__ __forceinline__ u32x4 fnv4(u32x4 a, u32x4 b) {
  return u32x4{fnv(a.x, b.x), fnv(a.y, b.y), fnv(a.z, b.z), fnv(a.w, b.w)};
}
__device__ __forceinline__ u32 fnv_reduce(u32x4 v) { return fnv(fnv(fnv(v.x, v.y), v.z), v.w); }

// Eight neighbouring lanes work on one hash at a time: lane t of the group holds
// mix words 4t..4t+3 and fetches bytes 16t..16t+15 of each 128-byte DAG item, so
// a group reads one whole item per access.  Four hashes of the group are in
// flight together to keep four independent gathers outstanding per lane.
struct EthashBody {
  static constexpr KernelId kId = K_ETHASH;
  using Args = EthashDevArgs;
  static constexpr bool kBarriers = false;
  static constexpr bool kFlat = false;  // one nonce per thread of the launch grid
  static constexpr int kGroup = 8, kParallel = 4, kAccesses = 64;

  template <class SB>
  static __device__ __forceinline__ void run(const Args &a, SB &sb, unsigned char *, unsigned) {
    // These waves spend most of their time waiting for DAG lines; whenever one of them can issue it goes first, and a
    // partner's arithmetic fills the slots that are left (no effect natively, where every wave has this priority).
    __builtin_amdgcn_s_setprio(3);
    const u32 gid = sb.bid * sb.nthreads + sb.tid;
    const u64 nonce = a.start_nonce + gid;
    const int lane_in_group = (int)(sb.tid & (kGroup - 1));
    const int mix_idx = lane_in_group & 3;

    u64 st[25];
    st[0] = a.header[0]; st[1] = a.header[1]; st[2] = a.header[2]; st[3] = a.header[3];
    st[4] = nonce;
    st[5] = 0x01ull;  // Keccak padding of a 40-byte message in a 72-byte rate
#pragma unroll
    for (int i = 6; i < 25; i++) st[i] = 0;
    st[8] = 0x8000000000000000ull;
    keccak_f1600(st);

    Words8 cmw;  // this lane's own mix digest, filled in when its turn comes
    u32 *cm = cmw.w;
#pragma unroll 1
    for (int i = 0; i < kGroup; i += kParallel) {
      u32x4 mix[kParallel];
      u32 init0[kParallel];
#pragma unroll
      for (int p = 0; p < kParallel; p++) {
        // Hash (i+p) of the group: its owner's 64-byte seed is spread over the eight lanes.
        u32 sh[16];
#pragma unroll
        for (int j = 0; j < 8; j++) {
          sh[2 * j] = __shfl((u32)st[j], i + p, kGroup);
          sh[2 * j + 1] = __shfl((u32)(st[j] >> 32), i + p, kGroup);
        }
        mix[p] = mix_idx == 0   ? u32x4{sh[0], sh[1], sh[2], sh[3]}
                 : mix_idx == 1 ? u32x4{sh[4], sh[5], sh[6], sh[7]}
                 : mix_idx == 2 ? u32x4{sh[8], sh[9], sh[10], sh[11]}
                                : u32x4{sh[12], sh[13], sh[14], sh[15]};
        init0[p] = sh[0];
      }
#pragma unroll 1
      for (u32 acc = 0; acc < (u32)kAccesses; acc += 4) {
        const int t = (int)((acc >> 2) & 7);  // the lane holding mix word (acc % 32)
#pragma unroll
        for (u32 b = 0; b < 4; b++) {
          u32 offset[kParallel];
#pragma unroll
          for (int p = 0; p < kParallel; p++) {
            const u32 x = fnv(init0[p] ^ (acc + b), mix[p][b]);
            const u32 o = a.pow2_mask ? (x & a.pow2_mask) : (x % a.n_items);
            offset[p] = __shfl(o, t, kGroup);
          }
          u32x4 item[kParallel];
#pragma unroll
          for (int p = 0; p < kParallel; p++) item[p] = __builtin_nontemporal_load(a.dag + (size_t)offset[p] * 8 + lane_in_group);
#pragma unroll
          for (int p = 0; p < kParallel; p++) mix[p] = fnv4(mix[p], item[p]);
        }
      }
#pragma unroll
      for (int p = 0; p < kParallel; p++) {
        const u32 r = fnv_reduce(mix[p]);
        u32 all[8];
#pragma unroll
        for (int j = 0; j < 8; j++) all[j] = __shfl(r, j, kGroup);
        if (i + p == lane_in_group) {
#pragma unroll
          for (int j = 0; j < 8; j++) cm[j] = all[j];
        }
      }
    }

    // keccak256(seed64 || cmix32): 96 bytes in a 136-byte rate
#pragma unroll
    for (int j = 0; j < 4; j++) st[8 + j] = ((u64)cm[2 * j + 1] << 32) | cm[2 * j];
    st[12] = 0x01ull;
#pragma unroll
    for (int i = 13; i < 25; i++) st[i] = 0;
    st[16] = 0x8000000000000000ull;
    keccak_f1600(st);
    if (bswap64(st[0]) <= a.target) {
      Words8 dg;
#pragma unroll
      for (int j = 0; j < 4; j++) { dg.w[2 * j] = (u32)st[j]; dg.w[2 * j + 1] = (u32)(st[j] >> 32); }
      record_hit(a.out, nonce, dg, cmw);
    }
  }
};

}  // namespace hfuse
