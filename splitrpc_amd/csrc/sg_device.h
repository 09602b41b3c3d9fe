// sg_device.h -- device-side building blocks of the gfx950 scatter-gather
// engine: wavefront copy of one run, wavefront reductions, response-header
// rewrite with one header byte per lane.
//
// gfx950 only: 64-wide wavefronts, DPP wave shifts.
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
constexpr uint32_t kStNotRule = 1u << 5;     // a fragment's length departs from the fragmenting rule
constexpr uint32_t kStSlotState = 1u << 6;   // an application slot was not in the state the call expects
constexpr uint32_t kStPoolFull = 1u << 7;    // more requests in flight than the reassembly pool holds
constexpr uint32_t kInvalidReq = 0xffffffffu; // owner field of a descriptor the kernels must skip

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(1))) u32_unaligned { uint32_t v; };
__device__ __forceinline__ uint32_t load32_any(const uint8_t *p)
{
  return reinterpret_cast<const u32_unaligned *>(p)->v;
}

// Payload chunks are touched once: read from a ring slot, written to a tensor
// (or the other way round) and not looked at again by this library.  The
// nontemporal hint on both sides keeps them from displacing each other in the
// caches; measured on the 32-batch gather it is worth 8 % (stores alone 5 %,
// loads alone -5 %), and a plain 16-byte-per-lane copy kernel gains the same.
__device__ __forceinline__ void store16_aligned(uint8_t *p, u32x4 v)
{
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}

__device__ __forceinline__ u32x4 load16_aligned(const uint8_t *p)
{
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

// Address of byte `off` of the running kernel's argument block.  A kernel with one by-value
// argument finds that argument at byte 0: a table inside it can then be indexed by a value
// known only at run time with one scalar load (indexing the by-value copy itself would have
// the compiler spill the table to private memory).
__device__ __forceinline__ const uint8_t *kernarg_at(size_t off)
{
  return reinterpret_cast<const uint8_t *>((uintptr_t)__builtin_amdgcn_kernarg_segment_ptr()) + off;
}

// Load through the scalar data cache: for wave-uniform addresses of data that
// NO wavefront of the running kernel writes (tables and cursors produced by an
// earlier kernel, ring headers in a kernel that only reads the ring).  The
// scalar cache is read-only here and is invalidated at kernel boundaries.
template <class T>
__device__ __forceinline__ T sload(const T *p)
{
  typedef const __attribute__((address_space(4))) T *cptr;
  return *(cptr)(uintptr_t)p;
}

// The same, issued where it stands: the optimizer may not sink it below a
// branch into the block that uses the value, so independent table reads placed
// side by side travel together instead of one round trip after the other.
template <class T>
__device__ __forceinline__ T sload_here(const T *p)
{
  typedef const volatile __attribute__((address_space(4))) T *cptr;
  return *(cptr)(uintptr_t)p;
}

// ---------------------------------------------------------------------------
// The bump-ring cursor of an arena
// ---------------------------------------------------------------------------
// A kernel that derives its offsets from the cursor cannot overwrite the word
// its other wavefronts are still reading.  Two ways round that:
//  * a one-workgroup kernel behind the copy kernel advances the cursor
//    (k_finish) -- 2 to 4 us of stream time per call, which is nothing to a call
//    of hundreds of thousands of wavefronts and a quarter of a call of one batch;
//  * the copy kernel advances the cursor itself ("self-advancing"): a context
//    keeps, beside the plain cursor word, TWO cells in one 64-byte line, the
//    live one being the one written last (its two-bit version is one ahead of
//    the other's).  Every wavefront takes the live cell, and exactly one thread
//    of the launch writes the successor into the OTHER cell, stamped with what
//    tells this launch from every other: the address of the queue it was
//    dispatched on and its dispatch id there.  A wavefront of the same launch
//    that already finds that stamp on the newer cell knows the cell for its own
//    launch's work and takes the other one; the next kernel finds a foreign
//    stamp and takes the new cell.  Nothing waits, nothing counts wavefronts.
//    The queue word becomes visible before the stamp (a fence between the two
//    stores; readers take a cell in one scalar load), so a cell that shows the
//    new version also shows the whole new stamp.  Finding the live cell costs a
//    wavefront two 8-dword scalar loads and some twenty scalar instructions
//    (the gather of 220672 fragments alone 104.2 -> 106.7 us), so the kernels
//    that do it are instances of their own (ADV) and the host picks them for
//    calls of up to 65536 wavefronts, the trailing kernel for larger ones.
// The plain word and the live cell hold the same value whenever no kernel that
// writes them is running: whoever advances the cursor writes both (the plain
// word is read by no wavefront of a self-advancing kernel, the cells by none of
// any other kernel).  Layout, in 64-bit words: cell 0 {value, queue, stamp,
// PLAIN WORD}, cell 1 {value, queue, stamp, unused}.  Callers of the
// allocation-free entry point bring a bare 64-bit word instead (`cells` false).
constexpr uint32_t kCurValue = 0, kCurQueue = 1, kCurStamp = 2, kCurPlain = 3, kCurCell = 4;
constexpr uint32_t kCurWords = 2 * kCurCell;
static_assert(kCurValue == 0 && kCurQueue == 1 && kCurStamp == 2 && kCurCell == 4, "cursor_take unpacks a cell by hand");

__device__ __forceinline__ uint32_t cursor_newer(uint64_t stamp0, uint64_t stamp1)
{
  return ((((uint32_t)stamp1 & 3u) - ((uint32_t)stamp0 & 3u)) & 3u) == 1u ? 1u : 0u;
}

// For kernels beside which nothing else reads or writes the cursor (k_finish, the copy kernel
// behind a descriptor pass): `p` is a context's cursor (cells) or a bare word.
__device__ __forceinline__ uint64_t cursor_get(const uint64_t *p, bool cells)
{
  return p[cells ? kCurPlain : 0u];
}
__device__ __forceinline__ void cursor_put(uint64_t *p, bool cells, uint64_t v)
{
  if (cells) {
    p[cursor_newer(p[kCurStamp], p[kCurCell + kCurStamp]) * kCurCell + kCurValue] = v;
    p[kCurPlain] = v;
  } else {
    p[0] = v;
  }
}

// What tells this launch from every other: the queue it was dispatched on and the index of its
// dispatch packet there, both handed to every wavefront in scalar registers.  (The dispatch id
// has no builtin of its own: the declaration names the compiler's intrinsic.)
extern "C" __device__ unsigned long long sg_dispatch_id(void) __asm("llvm.amdgcn.dispatch.id");
// `seq`: the calling context's count of calls, folded into the 16 bits a queue address leaves
// unused.  A queue that is destroyed and created again at the same address starts its dispatch
// ids over; the context's count goes on, so the launch that gets an old id back still does not
// take the last call's stamp for its own.  (Replays of one graph carry one count and differ by
// their dispatch ids.)
__device__ __forceinline__ uint64_t launch_queue(uint32_t seq)
{
  return (uint64_t)(uintptr_t)__builtin_amdgcn_queue_ptr() ^ ((uint64_t)seq << 48);
}
__device__ __forceinline__ uint64_t launch_stamp()
{
  return (uint64_t)sg_dispatch_id() << 2;  // the low two bits of a stamp are the cell's version
}

// The live value as a wavefront of a self-advancing kernel sees it (wave-uniform, through the
// scalar cache).  *live: the cell it came from, *stamp: that cell's stamp.
__device__ __forceinline__ uint64_t cursor_take(const uint64_t *p, uint32_t seq, uint32_t *live, uint64_t *stamp)
{
  // a cell is one 8-dword scalar load
  const u32x8 c0 = sload_here(reinterpret_cast<const u32x8 *>(p)), c1 = sload_here(reinterpret_cast<const u32x8 *>(p + kCurCell));
  const uint64_t v0 = (uint64_t)c0[1] << 32 | c0[0], q0 = (uint64_t)c0[3] << 32 | c0[2], s0 = (uint64_t)c0[5] << 32 | c0[4];
  const uint64_t v1 = (uint64_t)c1[1] << 32 | c1[0], q1 = (uint64_t)c1[3] << 32 | c1[2], s1 = (uint64_t)c1[5] << 32 | c1[4];
  // this launch's own write, once visible, is the newer cell: one comparison decides
  const uint32_t n = cursor_newer(s0, s1);
  const bool own = (n ? q1 : q0) == launch_queue(seq) && ((n ? s1 : s0) & ~3ull) == launch_stamp();
  const uint32_t l = own ? n ^ 1u : n;
  *live = l;
  *stamp = l ? s1 : s0;
  return l ? v1 : v0;
}

// The successor, by ONE thread of the launch.  (Vector stores: nothing is ever
// written through the scalar cache.)
__device__ __forceinline__ void cursor_advance(uint64_t *p, uint32_t seq, uint32_t live, uint64_t live_stamp, uint64_t value)
{
  uint64_t *cell = p + (live ^ 1u) * kCurCell;
  p[kCurPlain] = value;  // no wavefront of a self-advancing kernel reads the plain word
  cell[kCurValue] = value;
  cell[kCurQueue] = launch_queue(seq);
  __threadfence();
  __hip_atomic_store(cell + kCurStamp, launch_stamp() | ((live_stamp + 1u) & 3ull), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// (c + n * size) % cap for c < cap.
__device__ __forceinline__ uint64_t cursor_bump(uint64_t c, uint64_t n, uint64_t size, uint64_t cap)
{
  uint64_t t = n * size;
  if (t >= cap) t %= cap;  // a gather batch fits its arena; responses may lap theirs
  const uint64_t e = c + t;
  return e >= cap ? e - cap : e;
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

// Bytes [p, p+16) of the 32-byte window {lo, hi}, p = 4*Q + bs.
template <int Q>
__device__ __forceinline__ u32x4 window_q(u32x4 lo, u32x4 hi, uint32_t bs)
{
  const uint32_t D[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  u32x4 o;
#pragma unroll
  for (int j = 0; j < 4; j++)
    o[j] = __builtin_amdgcn_alignbyte(D[Q + j + 1 > 7 ? 7 : Q + j + 1], D[Q + j], bs);
  return o;
}

// The destination chunk a lane stores, from the aligned source chunk it loaded
// (`v`) and the one its upper neighbour loaded; p is the source phase 0..15.
__device__ __forceinline__ u32x4 realign(u32x4 v, uint32_t p)
{
  u32x4 nx;
#pragma unroll
  for (int j = 0; j < 4; j++) nx[j] = wave_shl1(v[j]);
  const uint32_t bs = p & 3u;
  switch (p >> 2) {
    case 0: return window_q<0>(v, nx, bs);
    case 1: return window_q<1>(v, nx, bs);
    case 2: return window_q<2>(v, nx, bs);
    default: return window_q<3>(v, nx, bs);
  }
}

// One run (a contiguous piece of payload) in the hands of one wavefront.
//
// Stores are 16-byte aligned: the destination decides the phase.  Loads are
// 16-byte ALIGNED too, whatever phase that leaves the source in: every lane
// loads one aligned source chunk per step (64 chunks = exactly eight 128-byte
// lines), takes its upper neighbour's chunk through a DPP wave shift and
// byte-aligns the 32-byte window into one destination chunk, so 64 loaded
// chunks yield 63 stored ones.  (A 16-byte load from an address that is not a
// multiple of 4 costs about an eighth of the achievable bandwidth.)  All loaded
// chunks hold at least one byte of the run, so nothing outside the run's own
// 16-byte-aligned hull is read.  The up-to-15 bytes before the first aligned
// store and after the last one move as single bytes on lanes 0..15 / 16..31.
//
// run_begin issues the edge-byte load and the loads of the first two steps
// (126 destination chunks, 2016 bytes); run_end realigns, stores and walks the
// rest.  A wavefront that begins several runs before ending the first keeps
// that many runs' loads in flight.
struct RunState {
  const uint8_t *src;
  uint8_t *dst;
  const uint8_t *sa;  // source of the first aligned store, rounded down to 16
  uint8_t *d;         // first aligned store
  uint32_t body;      // number of aligned 16-byte stores
  uint32_t lim;       // last source chunk to load (body when the phase is non-zero)
  uint32_t p;         // source phase
  uint32_t eoff;      // this lane's edge byte, if any
  uint32_t eb;
  bool edge;
  u32x4 v0, v1;
};

__device__ __forceinline__ void run_begin(RunState &r, const uint8_t *__restrict__ src,
                                          uint8_t *__restrict__ dst, uint32_t len, uint32_t lane)
{
  uint32_t head = (uint32_t)(-(uintptr_t)dst) & 15u;
  head = head < len ? head : len;
  const uint32_t body = (len - head) >> 4;
  const uint32_t tail = (len - head) & 15u;
  r.src = src;
  r.dst = dst;
  r.body = body;
  r.edge = false;
  r.eoff = 0;
  if (lane < 16) {
    r.edge = lane < head;
    r.eoff = lane;
  } else if (lane < 32) {
    r.edge = (lane - 16) < tail;
    r.eoff = head + (body << 4) + (lane - 16);
  }
  r.eb = 0;
  if (r.edge) r.eb = src[r.eoff];
  const uint8_t *s = src + head;
  r.d = dst + head;
  r.p = (uint32_t)(uintptr_t)s & 15u;
  r.sa = s - r.p;
  r.lim = r.p ? body : body - 1;  // body == 0: lim wraps, guarded below
  r.v0 = (u32x4){0, 0, 0, 0};
  r.v1 = (u32x4){0, 0, 0, 0};
  if (body) {
    if (lane <= r.lim) r.v0 = load16_aligned(r.sa + ((size_t)lane << 4));
    if (63u + lane <= r.lim) r.v1 = load16_aligned(r.sa + ((size_t)(63u + lane) << 4));
  }
}

// With CSUM returns this lane's share of the sum of the 16-bit little-endian
// words the run's bytes fall into, a byte's position in its word being the
// parity of its DESTINATION ADDRESS (packet offsets and addresses have the
// same parity: ring bases, slot sizes and header lengths are even).
//
// BROKEN: the destination is two pieces -- aligned chunks from number `brk` on, and the tail
// bytes, land `jump` bytes further (a fragment that runs from one tensor into the next, where
// the second tensor's share starts on a 16-byte boundary and the first one's share ends on a
// chunk boundary of the run): one run instead of two.
template <bool CSUM, bool BROKEN = false>
__device__ __forceinline__ uint32_t run_end(RunState &r, uint32_t lane, uint32_t brk = 0, int64_t jump = 0)
{
  uint32_t acc = 0;
  const u32x4 o0 = realign(r.v0, r.p);
  const u32x4 o1 = realign(r.v1, r.p);
  auto at = [&](uint32_t c) { return r.d + ((size_t)c << 4) + ((BROKEN && c >= brk) ? jump : (int64_t)0); };
  if (lane < 63 && lane < r.body) {
    store16_aligned(at(lane), o0);
    if (CSUM) acc += words_sum(o0);
  }
  if (lane < 63 && 63u + lane < r.body) {
    store16_aligned(at(63u + lane), o1);
    if (CSUM) acc += words_sum(o1);
  }
  for (uint32_t base = 126; base < r.body; base += 126) {
    const uint32_t c0 = base + lane, c1 = base + 63u + lane;
    u32x4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
    if (c0 <= r.lim) v0 = load16_aligned(r.sa + ((size_t)c0 << 4));
    if (c1 <= r.lim) v1 = load16_aligned(r.sa + ((size_t)c1 << 4));
    const u32x4 q0 = realign(v0, r.p);
    const u32x4 q1 = realign(v1, r.p);
    if (lane < 63 && c0 < r.body) {
      store16_aligned(at(c0), q0);
      if (CSUM) acc += words_sum(q0);
    }
    if (lane < 63 && c1 < r.body) {
      store16_aligned(at(c1), q1);
      if (CSUM) acc += words_sum(q1);
    }
  }
  if (r.edge) {
    // head bytes sit on lanes 0..15, tail bytes (behind the last aligned chunk) on lanes 16..31
    uint8_t *e = r.dst + r.eoff + ((BROKEN && lane >= 16) ? jump : (int64_t)0);
    *e = (uint8_t)r.eb;
    if (CSUM) acc += ((uintptr_t)e & 1u) ? (r.eb << 8) : r.eb;
  }
  return acc;
}

// Copy `len` bytes src -> dst with one wavefront.
template <bool CSUM>
__device__ __forceinline__ uint32_t copy_run(const uint8_t *__restrict__ src,
                                             uint8_t *__restrict__ dst, uint32_t len, uint32_t lane)
{
  RunState r;
  run_begin(r, src, dst, len, lane);
  return run_end<CSUM>(r, lane);
}

// A LONG run (jumbo frames) is cut into sub-runs of kPieceChunks destination
// chunks that different wavefronts (or one wavefront, several at a time) copy with
// the functions above: sub-run 0 is the head bytes plus the first
// kPieceChunks aligned chunks, every later one starts on a 16-byte destination
// boundary, the last one takes the tail bytes.  A sub-run's aligned source
// loads may reach into its neighbours' bytes -- which are bytes of the same run.
constexpr uint32_t kPieceChunks = 126;
constexpr uint32_t kPieceBytes = kPieceChunks * 16;

// How many sub-runs a run of at most `max_len` bytes is cut into.
__host__ __device__ inline uint32_t pieces_for(uint32_t max_len)
{
  const uint32_t chunks = (max_len >> 4) + 1;
  return (chunks + kPieceChunks - 1) / kPieceChunks;
}

// Offset and length of sub-run `piece` of a run of `len` bytes to `dst`;
// length 0 when the run has no such sub-run.
__device__ __forceinline__ void sub_run(const uint8_t *dst, uint32_t len, uint32_t piece, uint32_t *off,
                                        uint32_t *n)
{
  uint32_t head = (uint32_t)(-(uintptr_t)dst) & 15u;
  head = head < len ? head : len;
  const uint32_t start = piece == 0 ? 0 : head + piece * kPieceBytes;
  const uint32_t end = head + (piece + 1) * kPieceBytes;
  *off = start;
  *n = start >= len ? 0 : (end < len ? end : len) - start;
}

// Copy a whole long run with one wavefront, DEPTH sub-runs in flight at a time.
template <bool CSUM, int DEPTH>
__device__ __forceinline__ uint32_t copy_long_run(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                  uint32_t len, uint32_t lane)
{
  uint32_t acc = 0;
  for (uint32_t base = 0;; base += DEPTH) {
    RunState r[DEPTH];
    uint32_t n[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; k++) {
      uint32_t o;
      sub_run(dst, len, base + k, &o, &n[k]);
      if (n[k]) run_begin(r[k], src + o, dst + o, n[k], lane);
    }
#pragma unroll
    for (int k = 0; k < DEPTH; k++)
      if (n[k]) acc += run_end<CSUM>(r[k], lane);
    if (!n[DEPTH - 1]) break;
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
  uint32_t from_template;  // bytes come from a connection template: nothing was swapped, and the
                           // checksum fields keep the template's bytes unless a flag fills them
  uint32_t set_token;      // write `token` into bytes 42..49
  uint64_t token;
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

// The byte lane `lane` starts from: the incoming header's byte at the swapped
// position.  Split from hdr_finish so that a kernel can have this load in
// flight together with its payload loads.
__device__ __forceinline__ uint32_t hdr_fetch(const uint8_t *__restrict__ in, uint32_t lane, uint32_t hl,
                                              bool swap = true)
{
  uint32_t b = 0;
  if (lane < hl) b = in[swap ? hdr_src_index(lane) : lane];
  return b;
}

// Returns the final value of header byte `lane` (garbage on lanes >= hl) from
// the fetched byte.
// With l4_partial the finished UDP checksum is somebody else's business (the
// payload's sum is not known yet): the field is left zero and *l4_partial gets
// the sum of everything but the payload, unfolded.
__device__ __forceinline__ uint32_t hdr_finish(uint32_t b, uint32_t lane, const HdrFields &f,
                                               uint32_t payload_sum, uint32_t *l4_partial = nullptr)
{
  const uint32_t j = lane;
  const bool live = j < f.hl;

  const uint32_t L = (f.hl - 42u) + f.payload_len;
  const uint32_t tot = (28u + L) & 0xffffu;
  const uint32_t ulen = (8u + L) & 0xffffu;
  if (j == 16) b = tot >> 8;
  if (j == 17) b = tot & 0xffu;
  if (j == 38) b = ulen >> 8;
  if (j == 39) b = ulen & 0xffu;
  if (!f.from_template && (j == 24 || j == 25 || j == 40 || j == 41)) b = 0;  // swap_eth_hdr zeroes both sums
  if (f.set_token && j >= 42 && j < 50) b = (uint32_t)(f.token >> (8u * (j - 42u))) & 0xffu;
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
    const uint32_t s_ip = wave_sum((j >= 14 && j < 34 && j != 24 && j != 25) ? w : 0u);
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
      uint32_t c = 0;
      if (l4_partial) {
        *l4_partial = s;
      } else {
        s = fold16(fold16(s) + fold16(payload_sum));
        c = (~s) & 0xffffu;
        if (c == 0) c = 0xffffu;
      }
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

__device__ __forceinline__ uint32_t hdr_rewrite(const uint8_t *__restrict__ in, uint32_t lane,
                                                const HdrFields &f, uint32_t payload_sum)
{
  return hdr_finish(hdr_fetch(in, lane, f.hl), lane, f, payload_sum);
}


// ---- short frames: several frames per wavefront -----------------------------
// A frame of a few hundred bytes does not fill a wavefront: most lanes idle
// while the wavefront pays the full price in instructions and round trips.
// The functions below give a frame to a GROUP of L = 16 or 32 consecutive
// lanes, so that a wavefront moves 64 / L frames at once.  Everything a group
// works with (addresses, lengths, indices) lives in vector registers, the same
// value on every lane of the group; nothing here is wavefront-uniform.

// Sum over the 16 lanes of a row, left in every lane of the row: DPP adds, no LDS.
__device__ __forceinline__ uint32_t row_sum(uint32_t v)
{
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xb1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4e, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false);  // row_half_mirror
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false);  // row_mirror
  return v;
}

// Sum over the L lanes of a group (8: half a row, the first three steps of row_sum).
template <int L>
__device__ __forceinline__ uint32_t group_sum(uint32_t v)
{
  if (L == 8) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xb1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4e, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false);  // row_half_mirror
    return v;
  }
  v = row_sum(v);
  if (L == 32) v += __shfl_xor(v, 16, 64);
  return v;
}

// One run in the hands of a group of L lanes: the scheme of RunState above with
// L aligned source chunks per step yielding L - 1 destination chunks (the
// group's last lane has no upper neighbour of its own: the wave shift hands it
// a foreign lane's chunk, which it does not use).  Lanes 0..15 of the group
// carry one head byte and one tail byte each; the lanes of a group of 8 carry
// two of each (bytes gl and gl + 8).
template <int L>
struct GroupRun {
  const uint8_t *sa;
  uint8_t *d;
  uint8_t *dst;
  uint32_t body, lim, p;
  uint32_t head_b, tail_b, tail_off;
  uint32_t head_b2, tail_b2;  // L == 8 only
  bool has_head, has_tail, has_head2, has_tail2;
  u32x4 v0, v1;
};

template <int L>
__device__ __forceinline__ void group_run_begin(GroupRun<L> &r, const uint8_t *src, uint8_t *dst, uint32_t len,
                                                uint32_t gl)
{
  uint32_t head = (uint32_t)(-(uintptr_t)dst) & 15u;
  head = head < len ? head : len;
  const uint32_t body = (len - head) >> 4;
  const uint32_t tail = (len - head) & 15u;
  r.dst = dst;
  r.body = body;
  r.has_head = gl < head;
  r.has_tail = gl < tail;
  r.tail_off = head + (body << 4) + gl;
  r.head_b = r.has_head ? src[gl] : 0u;
  r.tail_b = r.has_tail ? src[r.tail_off] : 0u;
  r.has_head2 = L < 16 && gl + 8 < head;
  r.has_tail2 = L < 16 && gl + 8 < tail;
  r.head_b2 = r.has_head2 ? src[gl + 8] : 0u;
  r.tail_b2 = r.has_tail2 ? src[r.tail_off + 8] : 0u;
  const uint8_t *s = src + head;
  r.d = dst + head;
  r.p = (uint32_t)(uintptr_t)s & 15u;
  r.sa = s - r.p;
  r.lim = r.p ? body : body - 1;  // body == 0: lim wraps, guarded below
  r.v0 = (u32x4){0, 0, 0, 0};
  r.v1 = (u32x4){0, 0, 0, 0};
  if (body) {
    if (gl <= r.lim) r.v0 = load16_aligned(r.sa + ((size_t)gl << 4));
    if ((L - 1) + gl <= r.lim) r.v1 = load16_aligned(r.sa + ((size_t)((L - 1) + gl) << 4));
  }
}

// A run begun against a stand-in destination of the right phase (its loads are then under way
// before the real destination is known) gets its destination here ...
template <int L>
__device__ __forceinline__ void group_run_rebase(GroupRun<L> &r, uint8_t *dst)
{
  const ptrdiff_t head = r.d - r.dst;
  r.dst = dst;
  r.d = dst + head;
}

// ... or is called off: nothing is stored.
template <int L>
__device__ __forceinline__ void group_run_cancel(GroupRun<L> &r)
{
  r.body = 0;
  r.has_head = r.has_head2 = false;
  r.has_tail = r.has_tail2 = false;
}

// Returns this lane's share of the little-endian 16-bit word sum with CSUM.
// Every lane of the wavefront has to call this (the realignment shifts values
// across lanes); a group without a run passes body = 0 and no edge bytes.
template <int L, bool CSUM>
__device__ __forceinline__ uint32_t group_run_end(GroupRun<L> &r, uint32_t gl)
{
  uint32_t acc = 0;
  // the phase differs from group to group: realign() switches on it per lane
  const u32x4 o0 = realign(r.v0, r.p);
  const u32x4 o1 = realign(r.v1, r.p);
  if (gl < L - 1 && gl < r.body) {
    store16_aligned(r.d + ((size_t)gl << 4), o0);
    if (CSUM) acc += words_sum(o0);
  }
  if (gl < L - 1 && (L - 1) + gl < r.body) {
    store16_aligned(r.d + ((size_t)((L - 1) + gl) << 4), o1);
    if (CSUM) acc += words_sum(o1);
  }
  // longer runs: the wavefront keeps stepping while any of its groups has chunks left
  for (uint32_t base = 2 * (L - 1); __any(base < r.body); base += 2 * (L - 1)) {
    const uint32_t c0 = base + gl, c1 = base + (L - 1) + gl;
    u32x4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
    if (c0 <= r.lim && base < r.body) v0 = load16_aligned(r.sa + ((size_t)c0 << 4));
    if (c1 <= r.lim && base < r.body) v1 = load16_aligned(r.sa + ((size_t)c1 << 4));
    const u32x4 q0 = realign(v0, r.p);
    const u32x4 q1 = realign(v1, r.p);
    if (gl < L - 1 && c0 < r.body) {
      store16_aligned(r.d + ((size_t)c0 << 4), q0);
      if (CSUM) acc += words_sum(q0);
    }
    if (gl < L - 1 && c1 < r.body) {
      store16_aligned(r.d + ((size_t)c1 << 4), q1);
      if (CSUM) acc += words_sum(q1);
    }
  }
  if (r.has_head) {
    r.dst[gl] = (uint8_t)r.head_b;
    if (CSUM) acc += ((uintptr_t)(r.dst + gl) & 1u) ? (r.head_b << 8) : r.head_b;
  }
  if (r.has_tail) {
    r.dst[r.tail_off] = (uint8_t)r.tail_b;
    if (CSUM) acc += ((uintptr_t)(r.dst + r.tail_off) & 1u) ? (r.tail_b << 8) : r.tail_b;
  }
  if (L < 16) {
    if (r.has_head2) {
      r.dst[gl + 8] = (uint8_t)r.head_b2;
      if (CSUM) acc += ((uintptr_t)(r.dst + gl + 8) & 1u) ? (r.head_b2 << 8) : r.head_b2;
    }
    if (r.has_tail2) {
      r.dst[r.tail_off + 8] = (uint8_t)r.tail_b2;
      if (CSUM) acc += ((uintptr_t)(r.dst + r.tail_off + 8) & 1u) ? (r.tail_b2 << 8) : r.tail_b2;
    }
  }
  return acc;
}

// Response header of one frame on the first 16 lanes of a group, two 16-bit
// words per lane: lane j holds header bytes 4j .. 4j+3.  Every field of the
// header is a whole number of 16-bit words at an even offset, so the rewrite
// of hdr_finish above becomes word moves: word h comes from word hdr_src_word(h)
// of the incoming header (MACs, addresses, ports exchanged) or from word h of a
// template, length / routing / checksum words are overridden, and the sums run
// over the words as they lie in memory (little-endian), which yields the
// network-order checksums.  Same fields and flags as HdrFields.
__device__ __forceinline__ uint32_t hdr_src_word(uint32_t h)
{
  if (h < 3) return h + 3;
  if (h < 6) return h - 3;
  if (h == 13 || h == 14) return h + 2;
  if (h == 15 || h == 16) return h - 2;
  if (h == 17) return 18;
  if (h == 18) return 17;
  return h;
}

// W = words per lane: 2 on the first 16 lanes of a group of 16 or 32, 4 on the 8 lanes of a group of 8
// (lane j holds words W j .. W j + W - 1).
template <int W>
struct SmallHdr {
  uint32_t w[W];  // as fetched
};

template <int W>
__device__ __forceinline__ SmallHdr<W> small_hdr_fetch(const uint8_t *in, uint32_t j, uint32_t hl, bool swap, bool live)
{
  SmallHdr<W> h;
  const uint32_t n_words = hl >> 1;
  const uint16_t *w = reinterpret_cast<const uint16_t *>(in);  // rings and templates start at even addresses
#pragma unroll
  for (int k = 0; k < W; k++) {
    const uint32_t x = W * j + k;
    h.w[k] = (live && x < n_words) ? w[swap ? hdr_src_word(x) : x] : 0u;
  }
  return h;
}

__device__ __forceinline__ uint32_t bswap16(uint32_t v) { return ((v & 0xffu) << 8) | ((v >> 8) & 0xffu); }

// One header word's final value.
__device__ __forceinline__ uint32_t small_hdr_word(uint32_t v, uint32_t h, const HdrFields &f, uint32_t tot, uint32_t ulen)
{
  if (h == 8) v = bswap16(tot);
  if (h == 19) v = bswap16(ulen);
  if (!f.from_template && (h == 12 || h == 20)) v = 0;  // swap_eth_hdr zeroes both sums
  if (f.set_token && h >= 21 && h < 25) v = (uint32_t)(f.token >> (16u * (h - 21u))) & 0xffffu;
  if (f.ref64) {
    if (h == 25 || h == 26) v = 0;  // sock_perf_header &= 0xFFFFFFFF00000000
    if (h == 29) v = f.frag_idx & 0xffffu;
  } else {
    if (h == 25) v = f.frag_idx & 0xffffu;
    if (h == 26) v = f.num_frags & 0xffffu;
    if (h == 27) v = f.payload_len & 0xffffu;
    if (h == 28) v = f.payload_len >> 16;
  }
  return v;
}

// Finishes and stores the header of the group's frame at `out`.  `j` is the
// lane's index in its group; lanes 16.. of a 32-lane group take part in the
// sums only.  `live` says whether the group has a frame at all; payload_sum is
// the group-wide sum of the payload's little-endian words (full UDP checksum).
template <int L, int W>
__device__ __forceinline__ void small_hdr_finish(SmallHdr<W> s, uint8_t *out, uint32_t j, const HdrFields &f,
                                                 uint32_t payload_sum, bool live)
{
  static_assert(W * (L < 16 ? L : 16) == 32, "the header's 32 words over the lanes that hold it");
  const uint32_t n_words = f.hl >> 1;
  const uint32_t Lx = (f.hl - 42u) + f.payload_len;
  const uint32_t tot = (28u + Lx) & 0xffffu, ulen = (8u + Lx) & 0xffffu;
  uint32_t h[W], v[W];
  bool on[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    h[k] = W * j + k;
    on[k] = live && j < 32 / W && h[k] < n_words;
    v[k] = on[k] ? small_hdr_word(s.w[k], h[k], f, tot, ulen) : 0u;
  }
  const uint32_t kAnyCsum = 0x7u;  // IPV4 | PSEUDO | FULL
  if (f.flags & kAnyCsum) {
    auto in = [](uint32_t x, uint32_t a, uint32_t b) { return x >= a && x < b; };
    uint32_t t_ip = 0, t_addr = 0, t_pick = 0;
#pragma unroll
    for (int k = 0; k < W; k++) {
      t_ip += in(h[k], 7, 17) && h[k] != 12 ? v[k] : 0u;
      t_addr += in(h[k], 13, 17) ? v[k] : 0u;
      // word 7 = bytes 14, 15 (version/ihl first); word 11 = bytes 22, 23 (protocol second)
      t_pick += (h[k] == 7 ? (v[k] & 0xffu) : 0u) + (h[k] == 11 ? (v[k] & 0xff00u) : 0u);
    }
    const uint32_t s_ip = group_sum<L>(t_ip);
    const uint32_t s_addr = group_sum<L>(t_addr);
    const uint32_t pick = group_sum<L>(t_pick);
    const uint32_t b14 = pick & 0xffu, proto = pick >> 8;
    uint32_t udp = 0xffffffffu, ipc = 0xffffffffu;
    if (f.flags & (1u << 1)) {  // raw pseudo sum, reference style
      const uint32_t hdr_bytes = (f.flags & (1u << 3)) ? (b14 >> 4) * 4u : (b14 & 0xfu) * 4u;
      const uint32_t l = (tot - hdr_bytes) & 0xffffu;
      udp = fold16(s_addr + (proto << 8) + bswap16(l));
    }
    if (f.flags & (1u << 2)) {  // finished UDP checksum
      uint32_t t_l4 = 0;
#pragma unroll
      for (int k = 0; k < W; k++) t_l4 += (in(h[k], 17, 20) || in(h[k], 21, n_words)) ? v[k] : 0u;
      const uint32_t s_l4 = group_sum<L>(t_l4);
      uint32_t t = s_addr + (proto << 8) + bswap16(ulen) + s_l4;
      t = fold16(fold16(t) + fold16(payload_sum));
      udp = (~t) & 0xffffu;
      if (udp == 0) udp = 0xffffu;
    }
    if (f.flags & (1u << 0)) ipc = (~fold16(s_ip)) & 0xffffu;
#pragma unroll
    for (int k = 0; k < W; k++) {
      if (h[k] == 20 && udp != 0xffffffffu) v[k] = udp;
      if (h[k] == 12 && ipc != 0xffffffffu) v[k] = ipc;
    }
  }
  uint16_t *w = reinterpret_cast<uint16_t *>(out);
#pragma unroll
  for (int k = 0; k < W; k++)
    if (on[k]) w[h[k]] = (uint16_t)v[k];
}

// ---- the header as 16-bit words, one per lane -------------------------------
// For a kernel whose wavefront has ONE frame (k_scatter): lanes 0..31 hold the
// header's 16-bit words (29 of them with the 58-byte header, 32 with the
// 64-byte one).  Every field is a whole number of such words at an even
// offset, and everything that goes into a field is wavefront-uniform, so a
// field is written into its lane (v_writelane) and the few words a checksum
// needs are read out of their lanes (v_readlane): a couple of dozen
// instructions, where the byte-per-lane form above pays a compare and a select
// for every byte position and a cross-lane reduction for every sum.  Same
// fields, flags and results as hdr_finish.

// Sum over the wavefront, wavefront-uniform: row reductions by DPP, the four
// row totals added on the scalar side.
__device__ __forceinline__ uint32_t wave_sum_uniform(uint32_t v)
{
  v = row_sum(v);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 0) + (uint32_t)__builtin_amdgcn_readlane((int)v, 16) +
         (uint32_t)__builtin_amdgcn_readlane((int)v, 32) + (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
}

// Distance from header word h to the word it takes its value from when MACs,
// addresses and ports change places (words 0-2 <-> 3-5, 13-14 <-> 15-16,
// 17 <-> 18), three bits two's complement per word; words from 19 on stay.
__host__ __device__ constexpr uint64_t hdrw_delta_table()
{
  uint64_t t = 0;
  for (int h = 0; h < 19; h++) {
    int d = 0;
    if (h < 3) d = 3;
    else if (h < 6) d = -3;
    else if (h == 13 || h == 14) d = 2;
    else if (h == 15 || h == 16) d = -2;
    else if (h == 17) d = 1;
    else if (h == 18) d = -1;
    t |= (uint64_t)(d & 7) << (3 * h);
  }
  return t;
}

__device__ __forceinline__ uint32_t hdrw_src(uint32_t h)
{
  constexpr uint64_t kDelta = hdrw_delta_table();
  const uint32_t k = h < 19u ? h : 19u;  // bits 57.. of the table are zero
  const uint32_t code = (uint32_t)(kDelta >> (3u * k));
  return h + (uint32_t)((int32_t)(code << 29) >> 29);
}

// The word lane `lane` starts from (zero on lanes past the header).
__device__ __forceinline__ uint32_t hdrw_fetch(const uint8_t *__restrict__ in, uint32_t lane, uint32_t hl, bool swap)
{
  const uint16_t *w = reinterpret_cast<const uint16_t *>(in);  // rings and templates start at even addresses
  uint32_t v = 0;
  if (lane < (hl >> 1)) v = w[swap ? hdrw_src(lane) : lane];
  return v;
}

// v_writelane_b32: clang has no builtin of this name for the LLVM intrinsic, so the intrinsic
// is declared under its own name (the compiler then also places the wait states it needs)
extern "C" __device__ int sg_llvm_amdgcn_writelane(int value, int lane, int old) __asm("llvm.amdgcn.writelane.i32");

__device__ __forceinline__ uint32_t hdrw_put(uint32_t v, uint32_t word, uint32_t value)
{
  return (uint32_t)sg_llvm_amdgcn_writelane((int)value, (int)word, (int)v);
}

__device__ __forceinline__ uint32_t hdrw_get(uint32_t v, uint32_t word)
{
  return (uint32_t)__builtin_amdgcn_readlane((int)v, (int)word);
}

// Lengths, routing words and the token; both checksum words cleared after a swap.
__device__ __forceinline__ uint32_t hdrw_fields(uint32_t v, const HdrFields &f)
{
  const uint32_t L = (f.hl - 42u) + f.payload_len;
  const uint32_t tot = (28u + L) & 0xffffu, ulen = (8u + L) & 0xffffu;
  v = hdrw_put(v, 8, bswap16(tot));
  v = hdrw_put(v, 19, bswap16(ulen));
  if (!f.from_template) {  // swap_eth_hdr zeroes both sums
    v = hdrw_put(v, 12, 0);
    v = hdrw_put(v, 20, 0);
  }
  if (f.set_token) {
#pragma unroll
    for (uint32_t k = 0; k < 4; k++) v = hdrw_put(v, 21 + k, (uint32_t)(f.token >> (16u * k)) & 0xffffu);
  }
  if (f.ref64) {
    v = hdrw_put(v, 25, 0);  // sock_perf_header &= 0xFFFFFFFF00000000
    v = hdrw_put(v, 26, 0);
    v = hdrw_put(v, 29, f.frag_idx & 0xffffu);
  } else {
    v = hdrw_put(v, 25, f.frag_idx & 0xffffu);
    v = hdrw_put(v, 26, f.num_frags & 0xffffu);
    v = hdrw_put(v, 27, f.payload_len & 0xffffu);
    v = hdrw_put(v, 28, f.payload_len >> 16);
  }
  return v;
}

// This lane's share of the UDP checksum's sum over the header (UDP header
// without the checksum word, and everything behind it): to be added to the
// lane's payload sum before the wavefront-wide reduction.
__device__ __forceinline__ uint32_t hdrw_l4_share(uint32_t v, uint32_t lane, uint32_t hl)
{
  return (lane >= 17u && lane < (hl >> 1) && lane != 20u) ? v : 0u;
}

// Checksum words.  l4_sum: wavefront-uniform sum of the payload's words plus
// the lanes' hdrw_l4_share.  With l4_partial the finished UDP checksum is
// somebody else's business: the word is left zero and *l4_partial gets the
// pseudo-header's share of the sum, unfolded.
__device__ __forceinline__ uint32_t hdrw_csums(uint32_t v, const HdrFields &f, uint32_t l4_sum,
                                               uint32_t *l4_partial = nullptr)
{
  const uint32_t kAnyCsum = 0x7u;  // IPV4 | PSEUDO | FULL
  if (f.flags & kAnyCsum) {
    const uint32_t L = (f.hl - 42u) + f.payload_len;
    const uint32_t tot = (28u + L) & 0xffffu, ulen = (8u + L) & 0xffffu;
    const uint32_t w7 = hdrw_get(v, 7), w11 = hdrw_get(v, 11);
    const uint32_t s_addr = hdrw_get(v, 13) + hdrw_get(v, 14) + hdrw_get(v, 15) + hdrw_get(v, 16);
    const uint32_t b14 = w7 & 0xffu, proto = w11 >> 8;
    if (f.flags & (1u << 1)) {  // raw pseudo sum, reference style
      const uint32_t hdr_bytes = (f.flags & (1u << 3)) ? (b14 >> 4) * 4u : (b14 & 0xfu) * 4u;
      const uint32_t l = (tot - hdr_bytes) & 0xffffu;
      v = hdrw_put(v, 20, fold16(s_addr + (proto << 8) + bswap16(l)));
    }
    if (f.flags & (1u << 2)) {  // finished UDP checksum
      const uint32_t s = s_addr + (proto << 8) + bswap16(ulen);
      uint32_t c = 0;
      if (l4_partial) {
        *l4_partial = s;
      } else {
        c = (~fold16(fold16(s) + fold16(l4_sum))) & 0xffffu;
        if (c == 0) c = 0xffffu;
      }
      v = hdrw_put(v, 20, c);
    }
    if (f.flags & (1u << 0)) {  // finished IPv4 header checksum: words 7..16 without word 12
      const uint32_t s_ip = s_addr + w7 + hdrw_get(v, 8) + hdrw_get(v, 9) + hdrw_get(v, 10) + w11;
      v = hdrw_put(v, 12, (~fold16(s_ip)) & 0xffffu);
    }
  }
  return v;
}

__device__ __forceinline__ void hdrw_store(uint8_t *out, uint32_t lane, uint32_t hl, uint32_t v)
{
  if (lane < (hl >> 1)) reinterpret_cast<uint16_t *>(out)[lane] = (uint16_t)v;
}

}  // namespace sg
