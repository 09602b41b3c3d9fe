// sg_device.h -- device-side building blocks of the gfx950 scatter-gather
// engine: wavefront copy of one run, wavefront reductions, response-header
// rewrite with one header byte per lane.
//
// gfx950 only: 64-wide wavefronts, unaligned global access enabled (a 16-byte
// load from any byte address is one global_load_dwordx4).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sg {

constexpr uint32_t kWave = 64;
constexpr uint32_t kBlock = 256;             // 4 wavefronts per workgroup
constexpr uint32_t kWavesPerBlock = kBlock / kWave;
constexpr uint32_t kXcds = 8;                // XCDs of an MI355X; workgroups go round-robin over them

// status bits a kernel can raise
constexpr uint32_t kStBadSlot = 1u << 0;     // slot index beyond the ring
constexpr uint32_t kStBadLen = 1u << 1;      // fragment longer than a slot can hold
constexpr uint32_t kStBadSize = 1u << 2;     // request larger than its destination
constexpr uint32_t kStBadFrames = 1u << 3;   // response frame count disagrees with the fragmenting rule
constexpr uint32_t kStBadTable = 1u << 4;    // CSR table is not a gap-free tiling of the items
constexpr uint32_t kInvalidReq = 0xffffffffu; // owner field of a descriptor the kernels must skip

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(1))) u32x4_unaligned { u32x4 v; };

__device__ __forceinline__ u32x4 load16_any(const uint8_t *p)
{
  return reinterpret_cast<const u32x4_unaligned *>(p)->v;
}

struct __attribute__((packed, aligned(1))) u32_unaligned { uint32_t v; };
__device__ __forceinline__ uint32_t load32_any(const uint8_t *p)
{
  return reinterpret_cast<const u32_unaligned *>(p)->v;
}

__device__ __forceinline__ void store16_aligned(uint8_t *p, u32x4 v)
{
  *reinterpret_cast<u32x4 *>(p) = v;
}

// Sum of the eight 16-bit little-endian words of a 16-byte chunk.
__device__ __forceinline__ uint32_t words_sum(u32x4 v)
{
  uint32_t s = 0;
#pragma unroll
  for (int i = 0; i < 4; i++) s += (v[i] & 0xffffu) + (v[i] >> 16);
  return s;
}

__device__ __forceinline__ uint32_t wave_sum(uint32_t v)
{
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

__device__ __forceinline__ uint32_t wave_or(uint32_t v)
{
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v |= __shfl_xor(v, m, 64);
  return v;
}

__device__ __forceinline__ uint32_t fold16(uint32_t s)
{
  s = (s & 0xffffu) + (s >> 16);
  s = (s & 0xffffu) + (s >> 16);
  return s;
}

// Lane i receives lane i+1's value (lane 63 receives 0): DPP wave shift left
// by one, a GFX9-family cross-lane move that needs no LDS.
__device__ __forceinline__ uint32_t wave_shl1(uint32_t v)
{
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x130, 0xf, 0xf, false);
}

// Bytes [p, p+16) of the 32-byte window {lo, hi}; 0 < p < 16.
template <int Q>
__device__ __forceinline__ u32x4 funnel_q(u32x4 lo, u32x4 hi, uint32_t bs)
{
  const uint32_t D[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  u32x4 o;
#pragma unroll
  for (int j = 0; j < 4; j++)
    o[j] = __builtin_amdgcn_alignbyte(D[Q + j + 1 > 7 ? 7 : Q + j + 1], D[Q + j], bs);
  return o;
}

__device__ __forceinline__ u32x4 funnel(u32x4 lo, u32x4 hi, uint32_t p)
{
  const uint32_t bs = p & 3u;
  switch (p >> 2) {
    case 0: return funnel_q<0>(lo, hi, bs);
    case 1: return funnel_q<1>(lo, hi, bs);
    case 2: return funnel_q<2>(lo, hi, bs);
    default: return funnel_q<3>(lo, hi, bs);
  }
}

// N x 63 destination chunks starting at chunk `base`, source phase p != 0.
// Every lane loads one ALIGNED 16-byte source chunk per sub-step (64 chunks =
// exactly eight 128-byte lines), takes its upper neighbour's chunk through a
// DPP wave shift and funnels the two into the destination chunk, so 64 loaded
// chunks yield 63 stored ones.  The source chunks touched all hold at least
// one byte of the run, so nothing outside the run's own 16-byte-aligned hull
// is read.
template <int N, bool CSUM>
__device__ __forceinline__ uint32_t funnel_step(const uint8_t *__restrict__ sa, uint8_t *__restrict__ d,
                                                uint32_t base, uint32_t body, uint32_t p,
                                                uint32_t lane)
{
  u32x4 v[N];
  uint32_t acc = 0;
#pragma unroll
  for (int k = 0; k < N; k++) {
    const uint32_t c = base + 63u * k + lane;
    v[k] = (u32x4){0, 0, 0, 0};
    if (c <= body) v[k] = *reinterpret_cast<const u32x4 *>(sa + ((size_t)c << 4));
  }
#pragma unroll
  for (int k = 0; k < N; k++) {
    const uint32_t c = base + 63u * k + lane;
    u32x4 nx;
#pragma unroll
    for (int j = 0; j < 4; j++) nx[j] = wave_shl1(v[k][j]);
    const u32x4 o = funnel(v[k], nx, p);
    if (lane < 63 && c < body) {
      store16_aligned(d + ((size_t)c << 4), o);
      if (CSUM) acc += words_sum(o);
    }
  }
  return acc;
}

// Copy `len` bytes src -> dst with one wavefront.  Stores are 16-byte aligned
// (the destination decides the phase).  A source that is then at least
// 4-byte aligned is read with plain 16-byte loads; any other source phase is
// read with aligned loads and realigned in registers (funnel_step), because a
// 16-byte load from an address that is not a multiple of 4 costs about an
// eighth of the achievable bandwidth.  The up-to-15 bytes before the first
// aligned store and after the last one move as single bytes on lanes 0..15
// and 16..31.
// With CSUM the function also returns this lane's share of the sum of the
// 16-bit little-endian words the run's bytes fall into, a byte's position in
// its word being the parity of its DESTINATION ADDRESS (packet offsets and
// addresses have the same parity: ring bases, slot sizes and header lengths
// are even).
template <bool CSUM>
__device__ __forceinline__ uint32_t copy_run(const uint8_t *__restrict__ src,
                                             uint8_t *__restrict__ dst, uint32_t len, uint32_t lane)
{
  uint32_t acc = 0;
  uint32_t head = (uint32_t)(-(uintptr_t)dst) & 15u;
  head = head < len ? head : len;
  const uint32_t body = (len - head) >> 4;
  const uint32_t tail = (len - head) & 15u;

  // edge bytes
  bool edge = false;
  uint32_t eoff = 0;
  if (lane < 16) {
    edge = lane < head;
    eoff = lane;
  } else if (lane < 32) {
    edge = (lane - 16) < tail;
    eoff = head + (body << 4) + (lane - 16);
  }
  uint32_t eb = 0;
  if (edge) eb = src[eoff];

  const uint8_t *s = src + head;
  uint8_t *d = dst + head;
  const uint32_t p = (uint32_t)(uintptr_t)s & 15u;
  if ((p & 3u) == 0) {
    uint32_t c = lane;
    // four chunks in flight per lane while they last
    for (; c + 3 * kWave < body; c += 4 * kWave) {
      u32x4 v0 = load16_any(s + ((size_t)c << 4));
      u32x4 v1 = load16_any(s + ((size_t)(c + kWave) << 4));
      u32x4 v2 = load16_any(s + ((size_t)(c + 2 * kWave) << 4));
      u32x4 v3 = load16_any(s + ((size_t)(c + 3 * kWave) << 4));
      store16_aligned(d + ((size_t)c << 4), v0);
      store16_aligned(d + ((size_t)(c + kWave) << 4), v1);
      store16_aligned(d + ((size_t)(c + 2 * kWave) << 4), v2);
      store16_aligned(d + ((size_t)(c + 3 * kWave) << 4), v3);
      if (CSUM) acc += words_sum(v0) + words_sum(v1) + words_sum(v2) + words_sum(v3);
    }
    // then two at a time, the second one predicated
    for (; c < body; c += 2 * kWave) {
      const bool two = c + kWave < body;
      u32x4 v0 = load16_any(s + ((size_t)c << 4));
      u32x4 v1 = {0, 0, 0, 0};
      if (two) v1 = load16_any(s + ((size_t)(c + kWave) << 4));
      store16_aligned(d + ((size_t)c << 4), v0);
      if (two) store16_aligned(d + ((size_t)(c + kWave) << 4), v1);
      if (CSUM) acc += words_sum(v0) + words_sum(v1);
    }
  } else {
    const uint8_t *sa = s - p;
    uint32_t base = 0;
    for (; base + 126u < body; base += 252u) acc += funnel_step<4, CSUM>(sa, d, base, body, p, lane);
    for (; base < body; base += 126u) acc += funnel_step<2, CSUM>(sa, d, base, body, p, lane);
  }
  if (edge) {
    dst[eoff] = (uint8_t)eb;
    if (CSUM) acc += ((uintptr_t)(dst + eoff) & 1u) ? (eb << 8) : eb;
  }
  return acc;
}

// Byte-wise copy into / out of a bump-ring arena that is NOT mirrored, for a
// run that crosses the arena end.
__device__ __forceinline__ void copy_run_wrapped(const uint8_t *src, uint8_t *arena, uint64_t cap,
                                                 uint64_t off, uint32_t len, uint32_t lane,
                                                 bool into_arena, uint8_t *other)
{
  for (uint32_t i = lane; i < len; i += kWave) {
    uint64_t o = (off + i) % cap;
    if (into_arena) arena[o] = src[i];
    else other[i] = arena[o];
  }
}

// ---- response header rewrite ------------------------------------------------
// Lane j < hl produces byte j of the outgoing header from the header at `in`:
//   swap_eth_hdr (src/p2p_rpc.h:64-83): dst/src MAC, src/dst IP, src/dst port
//   exchanged, ip.check and udp.check zeroed;
//   routing fields as rr_set_hdr writes them (src/transport/
//   dpdk_transport_ng.h:129-131): token kept, seq_num / frag_idx = i, low half
//   of sock_perf_header cleared (REF64); num_frags and payload_len (BL58);
//   add_ip_udp_len (src/p2p_rpc.h:51-56): tot_len = 28 + L, udp.len = 8 + L,
//   L = RPC tail + payload bytes, big-endian;
//   add_udp_cksum (src/p2p_rpc.h:58-61, src/eth_common.h:92-130): raw folded
//   pseudo-header sum, not complemented, stored natively;
//   optional finished IPv4 header checksum (RFC 1071) and finished UDP
//   checksum (RFC 768; payload_sum is the wave-uniform sum of the payload's
//   little-endian 16-bit words).
// All sums run over little-endian words and are stored natively, which yields
// the network-order checksum (RFC 1071 section 2(B), byte-order independence).
struct HdrFields {
  uint32_t hl;          // 58 or 64
  uint32_t ref64;       // profile
  uint32_t flags;       // SG_F_*
  uint32_t frag_idx;
  uint32_t num_frags;
  uint32_t payload_len;
};

__device__ __forceinline__ uint32_t hdr_src_index(uint32_t j)
{
  if (j < 6) return j + 6;
  if (j < 12) return j - 6;
  if (j >= 26 && j < 30) return j + 4;
  if (j >= 30 && j < 34) return j - 4;
  if (j == 34 || j == 35) return j + 2;
  if (j == 36 || j == 37) return j - 2;
  return j;
}

// Returns the final value of header byte `lane` (garbage on lanes >= hl).
__device__ __forceinline__ uint32_t hdr_rewrite(const uint8_t *__restrict__ in, uint32_t lane,
                                                const HdrFields &f, uint32_t payload_sum)
{
  const uint32_t j = lane;
  const bool live = j < f.hl;
  uint32_t b = 0;
  if (live) b = in[hdr_src_index(j)];

  const uint32_t L = (f.hl - 42u) + f.payload_len;
  const uint32_t tot = (28u + L) & 0xffffu;
  const uint32_t ulen = (8u + L) & 0xffffu;
  if (j == 16) b = tot >> 8;
  if (j == 17) b = tot & 0xffu;
  if (j == 38) b = ulen >> 8;
  if (j == 39) b = ulen & 0xffu;
  if (j == 24 || j == 25 || j == 40 || j == 41) b = 0;
  if (f.ref64) {
    if (j >= 50 && j < 54) b = 0;                 // sock_perf_header &= 0xFFFFFFFF00000000
    if (j == 58) b = f.frag_idx & 0xffu;
    if (j == 59) b = (f.frag_idx >> 8) & 0xffu;
  } else {
    if (j == 50) b = f.frag_idx & 0xffu;
    if (j == 51) b = (f.frag_idx >> 8) & 0xffu;
    if (j == 52) b = f.num_frags & 0xffu;
    if (j == 53) b = (f.num_frags >> 8) & 0xffu;
    if (j >= 54 && j < 58) b = (f.payload_len >> (8u * (j - 54u))) & 0xffu;
  }
  if (!live) b = 0;

  const uint32_t w = (j & 1u) ? (b << 8) : b;  // contribution to a little-endian word sum
  const uint32_t kAnyCsum = 0x7u;              // IPV4 | PSEUDO | FULL
  if (f.flags & kAnyCsum) {
    const uint32_t s_ip = wave_sum((j >= 14 && j < 34) ? w : 0u);
    const uint32_t s_addr = wave_sum((j >= 26 && j < 34) ? w : 0u);
    const uint32_t b14 = __shfl(b, 14, 64);
    const uint32_t proto = __shfl(b, 23, 64);
    if (f.flags & (1u << 1)) {  // raw pseudo sum, reference style
      const uint32_t hdr_bytes = (f.flags & (1u << 3)) ? (b14 >> 4) * 4u : (b14 & 0xfu) * 4u;
      const uint32_t l = (tot - hdr_bytes) & 0xffffu;
      const uint32_t s = fold16(s_addr + (proto << 8) + (((l & 0xffu) << 8) | (l >> 8)));
      if (j == 40) b = s & 0xffu;
      if (j == 41) b = s >> 8;
    }
    if (f.flags & (1u << 2)) {  // finished UDP checksum
      const uint32_t s_l4 = wave_sum(((j >= 34 && j < 40) || (j >= 42 && j < f.hl)) ? w : 0u);
      uint32_t s = s_addr + (proto << 8) + (((ulen & 0xffu) << 8) | (ulen >> 8)) + s_l4;
      s = fold16(fold16(s) + fold16(payload_sum));
      uint32_t c = (~s) & 0xffffu;
      if (c == 0) c = 0xffffu;
      if (j == 40) b = c & 0xffu;
      if (j == 41) b = c >> 8;
    }
    if (f.flags & (1u << 0)) {  // finished IPv4 header checksum
      const uint32_t c = (~fold16(s_ip)) & 0xffffu;
      if (j == 24) b = c & 0xffu;
      if (j == 25) b = c >> 8;
    }
  }
  return b;
}

}  // namespace sg
