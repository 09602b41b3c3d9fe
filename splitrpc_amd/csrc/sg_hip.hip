// sg_hip.hip -- kernels and C ABI of the gfx950 scatter-gather engine.
//
// Three kernels carry a batch:
//   k_prep_*   one workgroup (or, for short requests, one wavefront) per
//              request: exclusive scan of the fragment lengths (-> offset of
//              every fragment inside its request, the running sum gather_skbs
//              keeps, src/p2p_rpc_sg_engine.h:22-43) and the request total.
//              Emits 16-byte run descriptors.  k_req_scan then scans the
//              request totals through the device-resident bump-ring cursor
//              (src/p2p_rpc_tring.h:27-33); with one size for all requests the
//              offsets are multiples and k_prep_* writes them itself.
//   k_gather   one wavefront per fragment run: ring slot payload -> tensor.
//   k_scatter  one wavefront per response frame: tensor -> TX slot payload,
//              header rewrite, checksums.
// When the caller declares one request size and the fragmenting rule, the
// descriptor pass is skipped: k_gather_rule and the FUSED form of k_scatter
// derive every offset themselves and hold the tables against the rule.
// Plus k_copy_runs / k_swap_hdrs for the per-request entry points and k_ra_*
// for sorting a burst of arrivals into requests (sg_hip_reassemble).
#include <hip/hip_runtime.h>

#include <errno.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <new>
#include <vector>

#include "../../include/sg_hip.h"
#include "sg_device.h"

using namespace sg;

namespace {
// A kernel refuses part of its input: the bits go into the device status word
// (later kernels of the call look at it and then move nothing) and a flag goes
// up in pinned host memory, where the host finds it after synchronizing
// without having to copy anything back.  The flag is a plain store of a
// constant: whoever writes, the value is the same.
__device__ __forceinline__ void refuse(uint32_t *status, volatile uint32_t *flag, uint32_t bits)
{
  atomicOr(status, bits);
  *flag = 1u;
}
}  // namespace

namespace {

// ---------------------------------------------------------------------------
// device-side argument blocks
// ---------------------------------------------------------------------------

struct AppDev {
  uint8_t *tensor_base[SG_MAX_TENSORS];
  uint64_t tensor_size[SG_MAX_TENSORS];
  uint32_t n_tensors;
  uint32_t mirrored;
  uint8_t *arena;
  uint64_t cap;
};

struct PrepArgs {
  // mode 0 (gather): lengths from item_len[] or from the slot headers
  // mode 1 (scatter): lengths from the fragmenting rule over sizes[] / fixed_size
  uint32_t mode;
  uint32_t n_req;
  const uint8_t *ring;
  uint32_t n_slots;
  uint32_t slot_size;
  uint32_t hl;
  uint32_t mtu;
  const uint32_t *item_slot;
  const uint32_t *item_len;
  const uint32_t *first;
  const uint64_t *sizes;
  uint64_t fixed_size;     // mode 1: response size when sizes == NULL
                           // mode 0: size every request must have (0: any)
  uint32_t n_items;
  uint32_t packed;
  uint32_t fixed_offsets;  // packed: request r starts at cursor + r * fixed_size, no scan needed
  uint64_t cap;
  uint64_t max_req_bytes;  // tensor-major: sum of tensor sizes
  u32x4 *desc;             // {slot, len, offset in request, request}
  uint64_t *req_size;
  uint64_t *req_off;
  // The bump-ring cursor is one device word.  The descriptor pass only reads
  // it and leaves the advanced value in *next_cursor; the copy kernel of the
  // same call, which does not read the cursor, commits it.
  const uint64_t *cursor;
  uint64_t *next_cursor;
  uint64_t *offsets_out;
  // mode 1: where each frame's header comes from, held against the RX ring here
  // so that a bad index refuses the batch before anything is written
  const uint32_t *hdr_src_slot;
  const uint32_t *hdr_src_req;  // or one header source per request
  uint32_t rx_n_slots;
  // Counts that live on the device (what sg_hip_reassemble left): [0] requests,
  // [1] items.  n_req and n_items above are then upper bounds the launch was
  // sized with.  nullptr: the bounds are the counts.
  const uint32_t *counts;
  // k_prep_group: where every workgroup leaves the sum of its requests' totals (for the tiled
  // scan of many requests, which then needs no launch of its own to total the tiles); or nullptr
  uint64_t *part;
  // What this pass leaves for a later call that wants to reuse its descriptors
  // (SG_F_REUSE_DESC): desc_tag = {gen, requests, items}.
  uint32_t *desc_tag;
  uint32_t gen;
  uint32_t *status;
  volatile uint32_t *status_flag;  // pinned host word: non-zero once any kernel refused something
};

// The counts a kernel works with: the host's, or the device's held against the
// host's bounds.  More requests on the device than the launch was sized for is
// refused by k_finish / the descriptor pass.
__device__ __forceinline__ uint32_t dev_count(const uint32_t *counts, uint32_t k, uint32_t bound)
{
  if (!counts) return bound;
  const uint32_t v = sload(counts + k);
  return v < bound ? v : bound;
}

__device__ __forceinline__ void prep_effective(PrepArgs &a)
{
  if (!a.counts) return;
  const uint32_t n = sload(a.counts);
  if (n > a.n_req) refuse(a.status, a.status_flag, kStBadSize);
  a.n_req = n < a.n_req ? n : a.n_req;
  // gather: the item count comes with the request count; scatter: it is where the frame table ends
  const uint32_t items = a.mode == 0 ? sload(a.counts + 1) : (a.n_req ? a.first[a.n_req] : 0u);
  if (a.mode == 0 && items > a.n_items) refuse(a.status, a.status_flag, kStBadSize);
  a.n_items = items < a.n_items ? items : a.n_items;
}

// Exclusive scan over the threads of a workgroup of BLOCK threads, built from
// wavefront scans (DPP/permute shuffles) and one LDS slot per wavefront.
template <int BLOCK>
__device__ __forceinline__ uint64_t block_exclusive_scan(uint64_t v, uint64_t *lds_wave_tot,
                                                         uint64_t *total)
{
  constexpr uint32_t kWaves = BLOCK / kWave;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wv = threadIdx.x / kWave;
  uint64_t inc = v;
#pragma unroll
  for (int d = 1; d < (int)kWave; d <<= 1) {
    uint64_t up = __shfl_up(inc, d, 64);
    if ((int)lane >= d) inc += up;
  }
  if (kWaves == 1) {
    *total = __shfl(inc, kWave - 1, 64);
    return inc - v;
  }
  if (lane == kWave - 1) lds_wave_tot[wv] = inc;
  __syncthreads();
  uint64_t base = 0, tot = 0;
#pragma unroll
  for (uint32_t i = 0; i < kWaves; i++) {
    uint64_t t = lds_wave_tot[i];
    if (i < wv) base += t;
    tot += t;
  }
  __syncthreads();
  *total = tot;
  return base + inc - v;
}

// Length and slot of item f of request r; raises status bits for what it refuses.
__device__ __forceinline__ void prep_item(const PrepArgs &a, uint32_t f, uint32_t i, uint64_t size,
                                          uint32_t *slot, uint32_t *len, uint32_t *bad)
{
  uint32_t s = a.item_slot[f];
  uint32_t l = 0;
  if (s >= a.n_slots) {
    *bad |= kStBadSlot;
    s = 0;
  } else if (a.mode == 0) {
    l = a.item_len ? a.item_len[f] : load32_any(a.ring + (size_t)s * a.slot_size + 54);
    if (l > a.slot_size - a.hl) {
      *bad |= kStBadLen;
      l = 0;
    }
  } else {
    // frame i carries min(remaining, mtu) (src/transport/dpdk_rx_tx.h:137-139)
    const uint64_t taken = (uint64_t)i * a.mtu;
    const uint64_t rem = taken < size ? size - taken : 0;
    l = (uint32_t)(rem <= a.mtu ? rem : a.mtu);
    if (a.hdr_src_slot && a.hdr_src_slot[f] >= a.rx_n_slots) *bad |= kStBadSlot;
  }
  *slot = s;
  *len = l;
}

// Checks on one request's slice of the CSR table and on its total; returns the
// (possibly emptied) item range.
__device__ __forceinline__ uint32_t prep_range(const PrepArgs &a, uint32_t r, uint32_t *f0,
                                               uint32_t *f1, uint64_t *size)
{
  uint32_t bad = 0;
  *f0 = a.first[r];
  *f1 = a.first[r + 1];
  // the table must tile [0, n_items) without gaps, or descriptors of an
  // earlier call would be taken for this one's
  if (*f0 > *f1 || *f1 > a.n_items || (r == 0 && *f0 != 0) ||
      (r == a.n_req - 1 && *f1 != a.n_items)) {
    bad |= kStBadTable;
    *f0 = *f1 = 0;
  }
  *size = 0;
  if (a.mode == 1) {
    *size = a.sizes ? a.sizes[r] : a.fixed_size;
    const uint64_t want = (*size + a.mtu - 1) / a.mtu;
    if (want != (uint64_t)(*f1 - *f0) || *size > 0xffffffffull) {
      bad |= kStBadFrames;
      *f0 = *f1 = 0;
      *size = 0;
    }
    if (a.hdr_src_req && a.hdr_src_req[r] >= a.rx_n_slots) bad |= kStBadSlot;
  }
  return bad;
}

// What one request's owner (a thread) publishes once the request total is known.
__device__ __forceinline__ void prep_finish(const PrepArgs &a, uint32_t r, uint64_t total, uint32_t bad)
{
  if (total > 0xffffffffull) bad |= kStBadSize;
  if (!a.packed && total > a.max_req_bytes) bad |= kStBadSize;
  if (a.packed && total > a.cap) bad |= kStBadSize;
  if (a.mode == 0 && a.fixed_size && total != a.fixed_size) bad |= kStBadSize;
  if (bad) refuse(a.status, a.status_flag, bad);
  a.req_size[r] = total;
  if (r == 0 && a.desc_tag) {
    a.desc_tag[0] = a.gen;
    a.desc_tag[1] = a.n_req;
    a.desc_tag[2] = a.n_items;
  }
  if (a.packed && a.fixed_offsets) {
    // bump ring with equal sizes: ret = base + off; off = (off + size) % capacity
    const uint64_t c0 = *a.cursor % a.cap;
    const uint64_t off = (c0 + (uint64_t)r * (a.fixed_size % a.cap)) % a.cap;
    a.req_off[r] = off;
    if (a.offsets_out) a.offsets_out[r] = off;
    if (r == a.n_req - 1) {
      const uint64_t end = (off + a.fixed_size) % a.cap;
      *a.next_cursor = end;
      if (a.offsets_out) a.offsets_out[a.n_req] = end;
    }
  }
}

// One workgroup of BLOCK threads per request: block-wide exclusive scan of the
// fragment lengths, all header reads of a pass in flight together.
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void k_prep_block(PrepArgs a)
{
  __shared__ uint64_t wave_tot[BLOCK / kWave];
  prep_effective(a);
  const uint32_t r = blockIdx.x;
  if (r >= a.n_req) return;
  uint32_t f0, f1;
  uint64_t size;
  uint32_t bad = prep_range(a, r, &f0, &f1, &size);
  uint64_t carry = 0;
  for (uint32_t base = f0; base < f1; base += BLOCK) {
    const uint32_t f = base + threadIdx.x;
    uint32_t len = 0, slot = 0;
    if (f < f1) prep_item(a, f, f - f0, size, &slot, &len, &bad);
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan<BLOCK>(len, wave_tot, &tot);
    if (f < f1) {
      u32x4 d = {slot, len, (uint32_t)(carry + ex), r};
      a.desc[f] = d;
    }
    carry += tot;
  }
  // fold the status bits of all threads into thread 0
  bad = wave_or(bad);
  if ((threadIdx.x & (kWave - 1)) == 0 && bad) refuse(a.status, a.status_flag, bad);
  if (threadIdx.x == 0) prep_finish(a, r, carry, 0);
}

// One wavefront per request (requests of at most a few dozen fragments).
__global__ __launch_bounds__(kBlock) void k_prep_wave(PrepArgs a)
{
  prep_effective(a);
  const uint32_t r = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (r >= a.n_req) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t f0, f1;
  uint64_t size;
  uint32_t bad = prep_range(a, r, &f0, &f1, &size);
  uint64_t carry = 0;
  for (uint32_t base = f0; base < f1; base += kWave) {
    const uint32_t f = base + lane;
    uint32_t len = 0, slot = 0;
    if (f < f1) prep_item(a, f, f - f0, size, &slot, &len, &bad);
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan<kWave>(len, nullptr, &tot);
    if (f < f1) {
      u32x4 d = {slot, len, (uint32_t)(carry + ex), r};
      a.desc[f] = d;
    }
    carry += tot;
  }
  bad = wave_or(bad);
  if (lane == 0) prep_finish(a, r, carry, bad);
}

// Several requests per wavefront, L = 16 or 32 lanes each (requests of a handful of fragments:
// with a wavefront per request most lanes idle and the launch is as many wavefronts' worth of
// dependent round trips -- table, header, scan -- as there are requests).  The scan runs over the
// L lanes of a group; a request of more than L fragments takes more steps, and the wavefront
// keeps stepping while any of its groups has fragments left.
template <int L>
__global__ __launch_bounds__(kBlock) void k_prep_group(PrepArgs a)
{
  constexpr uint32_t G = kWave / L;
  __shared__ uint64_t group_tot[kWavesPerBlock * G];
  prep_effective(a);
  const uint32_t lane = threadIdx.x & (kWave - 1), gl = lane & (L - 1);
  const uint32_t wave = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const uint32_t r = wave * G + lane / L;
  const bool live = r < a.n_req;
  uint32_t f0 = 0, f1 = 0, bad = 0;
  uint64_t size = 0;
  if (live) bad = prep_range(a, r, &f0, &f1, &size);
  uint64_t carry = 0;
  for (uint32_t base = f0; __any(base < f1); base += L) {
    const uint32_t f = base + gl;
    uint32_t len = 0, slot = 0;
    if (f < f1) prep_item(a, f, f - f0, size, &slot, &len, &bad);
    // inclusive scan over the group's lanes
    uint32_t inc = len;
#pragma unroll
    for (int d = 1; d < L; d <<= 1) {
      const uint32_t up = __shfl_up(inc, d, L);
      if ((int)gl >= d) inc += up;
    }
    if (f < f1) {
      u32x4 d = {slot, len, (uint32_t)(carry + (inc - len)), r};
      a.desc[f] = d;
    }
    carry += __shfl(inc, L - 1, L);
  }
#pragma unroll
  for (int m = L / 2; m >= 1; m >>= 1) bad |= __shfl_xor(bad, m, L);
  if (live && gl == 0) prep_finish(a, r, carry, bad);
  if (a.part) {
    // the workgroup's requests added up: kWavesPerBlock * G consecutive requests per entry
    if (gl == 0) group_tot[threadIdx.x / L] = live ? carry : 0;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint64_t t = 0;
#pragma unroll
      for (uint32_t k = 0; k < kWavesPerBlock * G; k++) t += group_tot[k];
      a.part[blockIdx.x] = t;
    }
  }
}

// Scan of the request totals through the bump ring:
//   ret = base + off; off = (off + size) % capacity   (src/p2p_rpc_tring.h:27-33)
// Up to kScanTile requests: one workgroup does it all (k_req_scan).  Beyond:
// one workgroup per tile totals its requests (k_req_scan_local), then every
// tile takes the sum of the totals before it as its base and scans from there
// (k_req_scan_add).
constexpr int kScanBlock = 1024;
constexpr int kScanPerThread = 4;
constexpr uint32_t kScanTile = kScanBlock * kScanPerThread;
// fewest requests behind one entry of the tile-total scratch (k_prep_group<32>: two per wavefront)
constexpr uint32_t kPartMin = 2 * kWavesPerBlock;

// Exclusive scan of one tile; returns this thread's prefix for its first
// request and leaves its requests' sizes in sz[].
__device__ __forceinline__ uint64_t scan_tile(const PrepArgs &a, uint32_t q0, uint64_t *sz,
                                              uint64_t *wave_tot, uint64_t *tot)
{
  uint64_t mine = 0;
#pragma unroll
  for (int k = 0; k < kScanPerThread; k++) {
    sz[k] = (q0 + k < a.n_req) ? a.req_size[q0 + k] : 0;
    mine += sz[k];
  }
  return block_exclusive_scan<kScanBlock>(mine, wave_tot, tot);
}

__device__ __forceinline__ void scan_emit(const PrepArgs &a, uint32_t q0, const uint64_t *sz, uint64_t off)
{
  // off < capacity on entry; every size <= capacity (checked by the descriptor pass)
#pragma unroll
  for (int k = 0; k < kScanPerThread; k++) {
    if (q0 + k < a.n_req) {
      a.req_off[q0 + k] = off;
      if (a.offsets_out) a.offsets_out[q0 + k] = off;
    }
    off += sz[k];
    if (off >= a.cap) off %= a.cap;
  }
}

// A gathered batch larger than its arena would lap itself: wavefronts of the
// first and of the last requests would then write the same bytes in no
// particular order.  Refused instead.
__device__ __forceinline__ void scan_check_batch(const PrepArgs &a, uint64_t batch_bytes)
{
  if (a.mode == 0 && batch_bytes > a.cap) refuse(a.status, a.status_flag, kStBadSize);
}

__global__ __launch_bounds__(kScanBlock) void k_req_scan(PrepArgs a)
{
  __shared__ uint64_t wave_tot[kScanBlock / kWave];
  prep_effective(a);
  uint64_t run = *a.cursor % a.cap, batch_bytes = 0;
  for (uint32_t base = 0; base < a.n_req; base += kScanTile) {
    const uint32_t q0 = base + threadIdx.x * kScanPerThread;
    uint64_t sz[kScanPerThread], tot;
    const uint64_t ex = scan_tile(a, q0, sz, wave_tot, &tot);
    scan_emit(a, q0, sz, (run + ex) % a.cap);
    run = (run + tot) % a.cap;
    batch_bytes += tot;
  }
  if (threadIdx.x == 0) {
    *a.next_cursor = run;
    if (a.offsets_out) a.offsets_out[a.n_req] = run;
    scan_check_batch(a, batch_bytes);
  }
}

// tile totals go to tile_tot[blockIdx.x]; the local prefixes are recomputed by k_req_scan_add
__global__ __launch_bounds__(kScanBlock) void k_req_scan_local(PrepArgs a, uint64_t *tile_tot)
{
  __shared__ uint64_t wave_tot[kScanBlock / kWave];
  const uint32_t q0 = blockIdx.x * kScanTile + threadIdx.x * kScanPerThread;
  uint64_t sz[kScanPerThread], tot;
  (void)scan_tile(a, q0, sz, wave_tot, &tot);
  if (threadIdx.x == 0) tile_tot[blockIdx.x] = tot;
}

// Every tile sums the totals of the tiles before it (a few values) for its base
// and scans again from there; the last tile also publishes the advanced cursor.
// The tiled scan behind k_prep_group, in one launch: the sizes before a tile are the sums the
// descriptor kernel's workgroups left (`per_part` requests each; a tile's worth of them is a few
// hundred values), so no launch is spent on totalling the tiles.
__global__ __launch_bounds__(kScanBlock) void k_req_scan_parts(PrepArgs a, uint32_t per_part, uint32_t n_tiles)
{
  __shared__ uint64_t wave_tot[kScanBlock / kWave];
  const bool is_last = blockIdx.x == n_tiles - 1;
  const uint32_t parts_before = blockIdx.x * (kScanTile / per_part);  // a tile is a whole number of parts
  uint64_t s = 0, before = 0;
  for (uint32_t q = threadIdx.x; q < parts_before; q += kScanBlock) s += a.part[q];
  (void)block_exclusive_scan<kScanBlock>(s, wave_tot, &before);
  const uint64_t c0 = *a.cursor % a.cap;
  const uint64_t tile_base = (c0 + before % a.cap) % a.cap;
  const uint32_t q0 = blockIdx.x * kScanTile + threadIdx.x * kScanPerThread;
  uint64_t sz[kScanPerThread], tot;
  const uint64_t ex = scan_tile(a, q0, sz, wave_tot, &tot);
  scan_emit(a, q0, sz, (tile_base + ex % a.cap) % a.cap);
  if (is_last && threadIdx.x == 0) {
    const uint64_t batch_bytes = before + tot;
    const uint64_t end = (c0 + batch_bytes % a.cap) % a.cap;
    *a.next_cursor = end;
    if (a.offsets_out) a.offsets_out[a.n_req] = end;
    scan_check_batch(a, batch_bytes);
  }
}

__global__ __launch_bounds__(kScanBlock) void k_req_scan_add(PrepArgs a, const uint64_t *tile_tot, uint32_t n_tiles)
{
  __shared__ uint64_t wave_tot[kScanBlock / kWave];
  const bool is_last = blockIdx.x == n_tiles - 1;
  const uint32_t upto = is_last ? n_tiles : blockIdx.x;  // the last tile needs the batch total too
  uint64_t before = 0, batch_bytes = 0;
  for (uint32_t base = 0; base < upto; base += kScanBlock) {
    const uint32_t t = base + threadIdx.x;
    const uint64_t v = t < upto ? tile_tot[t] : 0;
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan<kScanBlock>(v, wave_tot, &tot);
    (void)ex;
    batch_bytes += tot;
  }
  before = is_last ? batch_bytes - tile_tot[blockIdx.x] : batch_bytes;
  const uint64_t c0 = *a.cursor % a.cap;
  const uint64_t tile_base = (c0 + before % a.cap) % a.cap;
  const uint32_t q0 = blockIdx.x * kScanTile + threadIdx.x * kScanPerThread;
  uint64_t sz[kScanPerThread], tot;
  const uint64_t ex = scan_tile(a, q0, sz, wave_tot, &tot);
  scan_emit(a, q0, sz, (tile_base + ex % a.cap) % a.cap);
  if (is_last && threadIdx.x == 0) {
    const uint64_t end = (c0 + batch_bytes % a.cap) % a.cap;
    *a.next_cursor = end;
    if (a.offsets_out) a.offsets_out[a.n_req] = end;
    scan_check_batch(a, batch_bytes);
  }
}

// ---------------------------------------------------------------------------
// gather / scatter
// ---------------------------------------------------------------------------

// Which item a wavefront works on.  Workgroups are dealt round-robin to the
// eight XCDs, each with its own L2.  Runs of kXcdRun consecutive workgroups'
// worth of items are given to one XCD, so that neighbouring fragment runs --
// which share the cache lines at their common destination boundary -- meet in
// one L2, while all XCDs still walk the same region of memory together.
constexpr uint32_t kXcdRun = 32;
__device__ __forceinline__ uint32_t item_of_wave(bool remap)
{
  uint32_t g = blockIdx.x;
  if (remap) {
    const uint32_t xcd = g % kXcds, k = g / kXcds;
    g = ((k / kXcdRun) * kXcds + xcd) * kXcdRun + (k % kXcdRun);
  }
  return __builtin_amdgcn_readfirstlane(g * kWavesPerBlock + threadIdx.x / kWave);
}

// Advancing the cursor.  A copy kernel that derives its offsets from the
// bump-ring cursor cannot advance that cursor itself: its own wavefronts may
// still read it, and a second word to write into would need a device word
// saying which of the two is live -- with the same problem.  (Letting the
// wavefronts count themselves in or out with atomics so that the last one may
// write was built and measured: one returning atomic per workgroup costs the
// 32-batch gather 4 to 11 % -- the wavefront that waits for its ticket holds its
// registers that much longer.)  So the advance is the business of a one-workgroup
// kernel launched right behind the copy kernel, which also publishes slot
// states where the caller keeps them.  A recorded graph may therefore hold any
// number of calls.
struct FinishArgs {
  uint64_t *cursor;       // advanced by n_req * size modulo cap; nullptr: nothing to advance
  uint64_t size;
  uint64_t cap;
  uint32_t n_req;         // requests of the call, or their upper bound with `counts`
  const uint32_t *counts; // device-resident request count, or nullptr
  // Application slot states (the h_state words of the reference's app_rr pool,
  // src/p2p_rpc_app_rr.h:15-46): the n_req slots from *slot_idx on go from
  // `expect` to `publish`, and *slot_idx moves on by n_req (modulo n_states).
  uint32_t *state;        // nullptr: no slot ring
  uint32_t n_states;
  uint32_t *slot_idx;
  uint32_t expect, publish;
  uint32_t all_or_nothing;  // a refused batch publishes and advances nothing (descriptor pass)
  uint32_t *status;
  volatile uint32_t *status_flag;
};

__global__ __launch_bounds__(kBlock) void k_finish(FinishArgs a)
{
  const uint32_t refused = *a.status;  // what earlier kernels left
  __syncthreads();                     // read by every thread before this kernel adds to it
  uint32_t n = a.n_req;
  if (a.counts) {
    const uint32_t v = sload(a.counts);
    if (v > n && threadIdx.x == 0) refuse(a.status, a.status_flag, kStBadSize);  // the launch was sized for fewer
    n = v < n ? v : n;
  }
  if (a.all_or_nothing && refused) return;
  if (a.cursor && threadIdx.x == 0) {
    // bump ring with equal sizes: off = (off + size) % capacity, n_req times
    const uint64_t c = *a.cursor;
    *a.cursor = (c % a.cap + ((uint64_t)n * a.size) % a.cap) % a.cap;
  }
  if (a.state) {
    const uint32_t i0 = *a.slot_idx % a.n_states;
    uint32_t bad = 0;
    for (uint32_t k = threadIdx.x; k < n; k += kBlock) {
      uint32_t s = i0 + k % a.n_states;
      s = s >= a.n_states ? s - a.n_states : s;
      // the words may live in pinned host memory, where the worker's loop reads and writes them
      if (__hip_atomic_load(a.state + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != a.expect) bad = 1;
      __hip_atomic_store(a.state + s, a.publish, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    if (bad) refuse(a.status, a.status_flag, kStSlotState);
    __syncthreads();  // every thread has read *slot_idx
    if (threadIdx.x == 0) *a.slot_idx = (i0 + n % a.n_states) % a.n_states;
  }
}

// What the fused kernels need to derive a descriptor themselves when all
// requests (responses) have one size and are cut by the fragmenting rule:
// item f belongs to request f / per_req, is its fragment f % per_req, carries
// min(remaining, mtu) bytes and starts i * mtu bytes into the request; request
// r starts at cursor + r * size in the bump ring.
struct RuleArgs {
  const uint32_t *item_slot;
  const uint32_t *first;     // CSR table to hold against the rule
  uint64_t size;
  uint32_t mtu;
  uint32_t per_req;
  uint32_t n_req;
  uint32_t n_slots;
  uint32_t single_wrap;  // n_req * size <= capacity: a request offset wraps at most once
  // A short last frame per response goes to k_scatter_small: this kernel then takes
  // per_launch = per_req - 1 frames of every response (else per_launch == per_req).
  uint32_t per_launch;
  uint32_t div_mul, div_shift;  // item / per_req == (item * div_mul) >> div_shift for item < 2^27
  uint32_t lmul, lshift;        // the same for per_launch
  const uint64_t *cursor;  // read only here; k_finish advances it behind this kernel
  uint64_t *offsets_out;
};

struct GatherArgs {
  const u32x4 *desc;
  const uint64_t *req_off;
  const uint8_t *ring;
  uint32_t slot_size;
  uint32_t hl;
  uint32_t n_items;
  uint32_t remap;
  uint32_t pieces;  // wavefronts per fragment
  uint32_t *status;
  volatile uint32_t *status_flag;  // pinned host word: non-zero once any kernel refused something
  uint64_t *cursor;             // packed: wavefront 0 commits *next_cursor unless the batch was refused
  const uint64_t *next_cursor;
  const uint32_t *counts;       // device-resident counts ([0] requests, [1] items), or nullptr
  AppDev app;
};

// Descriptor of item `item` from the rule; publishes the request offset and, on
// the batch's last item, the advanced cursor.  Returns status bits.
__device__ __forceinline__ uint32_t rule_desc(const RuleArgs &g, const AppDev &app, uint32_t item,
                                              uint32_t n_items, uint32_t n_req, uint32_t lane, uint32_t *slot,
                                              uint32_t *len, uint32_t *off, uint32_t *r,
                                              uint32_t *i, uint64_t *req_off)
{
  uint32_t bad = 0;
  *r = (uint32_t)(((uint64_t)item * g.div_mul) >> g.div_shift);  // item / per_req
  *i = item - *r * g.per_req;
  // the three table reads are independent: asked for together
  *slot = sload_here(g.item_slot + item);
  const uint32_t first_r = sload_here(g.first + *r);
  uint64_t c0 = app.n_tensors == 0 ? sload_here(g.cursor) : 0;
  *off = *i * g.mtu;
  const uint64_t rem = g.size - *off;
  *len = (uint32_t)(rem <= g.mtu ? rem : g.mtu);
  if (*slot >= g.n_slots) bad |= kStBadSlot;
  if (*i == 0 && first_r != item) bad |= kStBadTable;
  *req_off = 0;
  if (app.n_tensors == 0) {
    if (c0 >= app.cap) c0 %= app.cap;  // only after a set_cursor beyond the capacity
    uint64_t o = c0 + (uint64_t)*r * g.size;
    if (g.single_wrap) o = o >= app.cap ? o - app.cap : o;  // n_req * size <= capacity
    else o %= app.cap;
    *req_off = o;
    if (lane == 0) {
      if (*i == 0 && g.offsets_out) g.offsets_out[*r] = *req_off;
      if (item == n_items - 1 && g.offsets_out) {
        uint64_t end = *req_off + g.size;  // size <= capacity
        end = end >= app.cap ? end - app.cap : end;
        g.offsets_out[n_req] = end;
      }
    }
  }
  return bad;
}

// Move [off, off+len) of request r's byte stream between a packet payload and
// the application buffers.  TO_APP: packet -> app.  One copy_run call site:
// the packed arena is walked as a single piece, tensor-major buffers as up to
// SG_MAX_TENSORS pieces.
template <bool TO_APP, bool CSUM>
__device__ __forceinline__ uint32_t move_run(const AppDev &app, uint64_t req_off, uint32_t r,
                                             uint32_t off, uint8_t *pkt, uint32_t len, uint32_t lane)
{
  uint32_t acc = 0;
  const bool packed = app.n_tensors == 0;
  uint8_t *packed_ptr = nullptr;
  if (packed) {
    const uint64_t o = req_off + off;  // < 2 * cap
    if ((uint64_t)off + len > app.cap) return 0;  // request larger than the arena: refused elsewhere
    if (!app.mirrored && o < app.cap && o + len > app.cap) {
      // a run that crosses the end of an arena that is not mapped twice
      copy_run_wrapped(pkt, app.arena, app.cap, o, len, lane, TO_APP, pkt);
      if (CSUM) {
        for (uint32_t i = lane; i < len; i += kWave) {
          uint32_t b = pkt[i];  // this lane wrote it
          acc += ((uintptr_t)(pkt + i) & 1u) ? (b << 8) : b;
        }
      }
      return acc;
    }
    packed_ptr = app.arena + ((!app.mirrored && o >= app.cap) ? o - app.cap : o);
  }
  const uint32_t n_pieces = packed ? 1u : app.n_tensors;
  uint64_t t0 = 0;
  uint32_t done = 0;
  for (uint32_t t = 0; t < n_pieces && done < len; t++) {
    uint8_t *p;
    uint32_t n;
    if (packed) {
      p = packed_ptr;
      n = len;
    } else {
      const uint64_t t1 = t0 + app.tensor_size[t];
      const uint64_t cur = (uint64_t)off + done;
      t0 = t1;
      if (cur >= t1) continue;
      const uint64_t room = t1 - cur;
      n = room < (uint64_t)(len - done) ? (uint32_t)room : (len - done);
      p = app.tensor_base[t] + (uint64_t)r * app.tensor_size[t] + (cur - (t1 - app.tensor_size[t]));
    }
    acc += TO_APP ? copy_run<CSUM>(pkt + done, p, n, lane) : copy_run<CSUM>(p, pkt + done, n, lane);
    done += n;
  }
  return acc;
}

// Keeps a kernel argument in a scalar register from this point on.  Placed on
// every argument the hot path needs, at the top of a kernel, it makes the
// compiler fetch them all in one burst of scalar loads instead of one
// dependent round trip per first use.
#define SG_PIN(x) asm volatile("" ::"s"(x))

// Where [off, off+len) of request r's byte stream lives when that is ONE
// contiguous piece of application memory; false when it is not (a run that
// crosses the end of an arena mapped once, or a tensor boundary).
__device__ __forceinline__ bool plain_target(const AppDev &app, uint64_t req_off, uint32_t r,
                                             uint32_t off, uint32_t len, uint8_t **to)
{
  if (app.n_tensors == 0) {
    if ((uint64_t)off + len > app.cap) return false;
    uint64_t o = req_off + off;  // < 2 * capacity
    if (!app.mirrored) {
      if (o >= app.cap) o -= app.cap;
      else if (o + len > app.cap) return false;
    }
    *to = app.arena + o;
    return true;
  }
  uint64_t t0 = 0;
  for (uint32_t t = 0; t < app.n_tensors; t++) {
    const uint64_t t1 = t0 + app.tensor_size[t];
    if (off < t1) {
      if ((uint64_t)off + len > t1) return false;
      *to = app.tensor_base[t] + (uint64_t)r * app.tensor_size[t] + (off - t0);
      return true;
    }
    t0 = t1;
  }
  return false;
}

// Where byte `pos` of request r's stream lives, whatever the layout (the slow
// way, for the rare frame that straddles an arena end or a tensor boundary).
__device__ __forceinline__ uint8_t *app_byte(const AppDev &app, uint64_t req_off, uint32_t r, uint64_t pos)
{
  if (app.n_tensors == 0) return app.arena + (req_off + pos) % app.cap;
  uint64_t t0 = 0;
  for (uint32_t t = 0; t < app.n_tensors; t++) {
    if (pos < t0 + app.tensor_size[t]) return app.tensor_base[t] + (uint64_t)r * app.tensor_size[t] + (pos - t0);
    t0 += app.tensor_size[t];
  }
  return nullptr;
}

// [off, off+len) of request r's byte stream when it starts in one tensor-major
// buffer and ends in the next: the two pieces.  False for anything else.
__device__ __forceinline__ bool two_tensor_target(const AppDev &app, uint32_t r, uint32_t off, uint32_t len,
                                                  uint8_t **to_a, uint32_t *len_a, uint8_t **to_b)
{
  uint64_t t0 = 0;
  for (uint32_t t = 0; t + 1 < app.n_tensors; t++) {
    const uint64_t t1 = t0 + app.tensor_size[t];
    if (off < t1) {
      if ((uint64_t)off + len <= t1 || (uint64_t)off + len > t1 + app.tensor_size[t + 1]) return false;
      *to_a = app.tensor_base[t] + (uint64_t)r * app.tensor_size[t] + (off - t0);
      *len_a = (uint32_t)(t1 - off);
      *to_b = app.tensor_base[t + 1] + (uint64_t)r * app.tensor_size[t + 1];
      return true;
    }
    t0 = t1;
  }
  return false;
}

// Gather from descriptors written by the descriptor pass.  One wavefront per
// fragment piece: a fragment longer than kPieceChunks chunks is spread over
// `pieces` consecutive wavefronts.  (Several fragments per wavefront were
// measured too: two cost 2 %, three 13 % on 1400-byte fragments -- the number
// of wavefronts in flight is what covers the HBM latency.)
template <bool LONG>
__global__ __launch_bounds__(kBlock) void k_gather(GatherArgs a)
{
  const u32x4 *desc = a.desc;
  const uint64_t *req_off = a.req_off;
  const uint8_t *ring = a.ring;
  const uint32_t slot_size = a.slot_size, hl = a.hl, remap = a.remap;
  const uint32_t pieces = a.pieces;
  const uint32_t *status = a.status;
  const uint32_t *counts = a.counts;
  uint32_t n_items = a.n_items;
  SG_PIN(desc); SG_PIN(req_off); SG_PIN(ring); SG_PIN(slot_size); SG_PIN(hl); SG_PIN(n_items);
  SG_PIN(remap); SG_PIN(status); SG_PIN(pieces); SG_PIN(counts);
  if (counts) n_items = dev_count(counts, 1, n_items);
  const uint32_t w = item_of_wave(remap != 0);
  const uint32_t item = LONG ? w / pieces : w;
  const uint32_t piece = LONG ? w - item * pieces : 0;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  // this kernel does not read the cursor: the value the descriptor pass left is committed here
  // (a batch of no requests at all has left none)
  if (w == 0 && lane == 0 && a.cursor && !sload(status) && (!counts || sload(counts)))
    *a.cursor = sload(a.next_cursor);
  if (item >= n_items) return;
  const u32x4 d = sload_here(desc + item);  // asked for together with the status word
  if (sload_here(status)) return;           // the descriptor pass refused the batch: move nothing
  if (d[1] == 0 || d[3] == kInvalidReq) return;
  const uint64_t ro = a.app.n_tensors == 0 ? sload(req_off + d[3]) : 0;
  uint8_t *pkt = const_cast<uint8_t *>(ring) + (size_t)d[0] * slot_size + hl;
  uint8_t *to;
  if (plain_target(a.app, ro, d[3], d[2], d[1], &to)) {
    if (LONG) {
      uint32_t o, n;
      sub_run(to, d[1], piece, &o, &n);
      if (n) copy_run<false>(pkt + o, to + o, n, lane);
    } else {
      copy_run<false>(pkt, to, d[1], lane);
    }
  } else if (piece == 0) {
    move_run<true, false>(a.app, ro, d[3], d[2], pkt, d[1], lane);
  }
}

// Where the bytes of fragment i of every request go, several tensor-major buffers:
// request r's share of the fragment starts at base + r * stride.
struct FragPlan {
  uint64_t base_a, base_b;      // tensor base + offset inside the request's share (b: the next tensor's base)
  uint32_t stride_a, stride_b;  // bytes per request of the tensor(s)
  uint32_t len_a;               // bytes that go to the first tensor
  uint32_t kind;                // 0: one tensor, 1: two tensors, 2: more (general path)
};
constexpr uint32_t kPlanMax = 8;
static_assert(sizeof(FragPlan) == 32, "a plan entry is one 8-dword scalar load");

// Gather without a descriptor pass: all requests have `size` bytes cut by the
// fragmenting rule, so a wavefront derives its descriptor from its item
// number (item f belongs to request f / per_req, is its fragment f % per_req,
// carries min(remaining, mtu) bytes and starts i * mtu bytes into the request;
// request r starts at cursor + r * size in the bump ring) and holds the
// fragment's real length against the rule.
struct GatherRuleArgs {
  // hot: what a wavefront needs before its first payload load
  const uint8_t *ring;
  const uint32_t *frag_slot;
  uint8_t *dst;               // arena (packed) or the tensor (one tensor-major buffer)
  const uint64_t *cursor;     // packed only; read only here, k_finish advances it behind this kernel
  uint64_t size;
  uint64_t cap;               // packed: arena capacity; 0: tensor-major
  uint32_t n_items;
  uint32_t per_req;
  uint32_t div_mul, div_shift;  // item / per_req == (item * div_mul) >> div_shift for item < 2^27
  // A short last fragment per request goes to k_gather_small: this kernel then takes
  // per_launch = per_req - 1 fragments of every request (else per_launch == per_req);
  // lmul / lshift divide by per_launch as div_mul / div_shift divide by per_req.
  uint32_t per_launch, lmul, lshift;
  uint32_t period, pmul, pshift;  // wavefronts per turn of full and remainder work, and the division by it
  uint32_t mtu;
  uint32_t slot_size;
  uint32_t hl;
  uint32_t n_slots;
  uint32_t pieces;            // wavefronts per fragment
  uint32_t opts;  // kOptRemap | kOptMirrored | kOptMultiTensor | kOptHdrChunk
  // warm
  uint32_t n_req;
  const uint32_t *frag_len;
  const uint32_t *first;
  uint64_t *offsets_out;
  const uint32_t *counts;     // device-resident counts ([0] requests, [1] fragments), or nullptr
  uint32_t *status;
  volatile uint32_t *status_flag;  // pinned host word: non-zero once any kernel refused something
  AppDev app;  // consulted for several tensor-major buffers only
  // Several tensor-major buffers: where fragment i of a request lands depends on i alone (all
  // requests have one size), so the host walks the tensors once per fragment index and the
  // wavefront reads one entry instead of walking them itself.  n_plan == 0: no plan (too many
  // fragments per request, or tensors of 4 GiB and more per request).
  uint32_t n_plan;
  uint32_t plan_pad;
  FragPlan plan[kPlanMax];
};
constexpr uint32_t kOptRemap = 1u, kOptMirrored = 2u, kOptMultiTensor = 8u;
// slots start at 16-byte aligned addresses: the header's length field can be read as part of
// the aligned chunk at byte 48 (a ring only has to start at an even address)
constexpr uint32_t kOptHdrChunk = 16u;
constexpr uint32_t kOptSmallLast = 32u;  // the last fragment of every request is left to k_gather_small

template <int L>
__device__ __forceinline__ void gather_small_wave(const GatherRuleArgs &a, uint32_t wave);

// SMALL: lanes per remainder fragment (16 or 32) when the last fragment of every
// request is short -- the wavefronts behind those of the full fragments then move
// 64 / SMALL remainder fragments each, in the same launch (a launch of their own
// would be all latency: tens of megabytes at most); 0: no such wavefronts.
template <bool LONG, int SMALL>
__global__ __launch_bounds__(kBlock) void k_gather_rule(GatherRuleArgs a)
{
  const uint8_t *ring = a.ring;
  const uint32_t *frag_slot = a.frag_slot;
  uint8_t *dst = a.dst;
  const uint64_t *cursor_in = a.cursor;
  const uint64_t size = a.size, cap = a.cap;
  const uint32_t per_req = a.per_req, mtu = a.mtu, slot_size = a.slot_size;
  const uint32_t hl = a.hl, n_slots = a.n_slots, pieces = a.pieces, opts = a.opts;
  const uint32_t div_mul = a.div_mul, div_shift = a.div_shift;
  const uint32_t *counts = a.counts;
  uint32_t n_items = a.n_items, n_req = a.n_req;
  SG_PIN(ring); SG_PIN(frag_slot); SG_PIN(dst); SG_PIN(cursor_in); SG_PIN(size); SG_PIN(cap);
  SG_PIN(n_items); SG_PIN(per_req); SG_PIN(mtu); SG_PIN(slot_size); SG_PIN(hl); SG_PIN(n_slots);
  SG_PIN(pieces); SG_PIN(opts); SG_PIN(div_mul); SG_PIN(div_shift); SG_PIN(counts);
  if (counts) {
    // counts left on the device by the reassembly: the launch was sized for n_req requests at most
    n_req = dev_count(counts, 0, n_req);
    n_items = n_req * per_req;
  }

  uint32_t w = item_of_wave((opts & kOptRemap) != 0);
  const uint32_t pl = a.per_launch;
  if (SMALL) {
    // Wavefronts of the two kinds are dealt in turns: after the period - 1 wavefronts of the full
    // fragments of 64 / SMALL requests comes the one that moves those requests' remainders.  The
    // short-fragment wavefronts are bound by their arithmetic, the others by memory: side by side
    // on a CU they overlap, one kind after the other they would not.
    const uint32_t blk = (uint32_t)(((uint64_t)w * a.pmul) >> a.pshift);
    const uint32_t j = w - blk * a.period;
    if (j == a.period - 1) {
      gather_small_wave<(SMALL ? SMALL : 16)>(a, blk);
      return;
    }
    w = blk * (a.period - 1) + j;
    if (w >= n_req * pl * (LONG ? pieces : 1u)) return;
  }
  uint32_t item = LONG ? w / pieces : w;
  const uint32_t piece = LONG ? w - item * pieces : 0;
  // division by the fragments per request as a multiplication the host prepared (a division of
  // two scalars is some twenty scalar instructions, and the scalar unit is the busiest here)
  uint32_t r, i;
  if (SMALL) {
    r = (uint32_t)(((uint64_t)item * a.lmul) >> a.lshift);
    i = item - r * pl;
    item = r * per_req + i;
  } else {
    if (item >= n_items) return;
    r = (uint32_t)(((uint64_t)item * div_mul) >> div_shift);
    i = item - r * per_req;
  }
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t slot = sload(frag_slot + item);
  uint64_t c0 = cap ? sload(cursor_in) : 0;
  const uint32_t off = i * mtu;
  const uint32_t rem = (uint32_t)size - off;  // sizes are below 4 GiB (checked by the host)
  const uint32_t len = rem <= mtu ? rem : mtu;
  uint8_t *pkt = const_cast<uint8_t *>(ring) + (size_t)slot * slot_size;

  uint64_t ro = 0;
  bool plain = !(opts & kOptMultiTensor);
  uint8_t *to = nullptr;
  uint8_t *to_a = nullptr, *to_b = nullptr;
  uint32_t len_a = 0, plan_kind = 3;  // 3: no plan, the tensors are walked here
  if (cap) {
    // bump ring with equal sizes: request r starts at (cursor + r * size) % capacity
    if (c0 >= cap) c0 %= cap;  // only after a set_cursor beyond the capacity
    ro = c0 + (uint64_t)r * size;
    ro = ro >= cap ? ro - cap : ro;  // the batch fits the arena (checked by the host): one wrap at most
    if (lane == 0 && piece == 0 && a.offsets_out) {
      if (i == 0) a.offsets_out[r] = ro;
      if (item == n_items - 1) {
        uint64_t end = ro + size;  // size <= capacity
        a.offsets_out[n_req] = end >= cap ? end - cap : end;
      }
    }
    uint64_t o = ro + off;  // < 2 * capacity
    if (!(opts & kOptMirrored)) {
      if (o >= cap) o -= cap;
      else if (o + len > cap) plain = false;  // crosses the end of an arena mapped once
    }
    to = dst + o;
  } else if (opts & kOptMultiTensor) {
    // tensor-major buffers: a fragment inside one tensor still takes the fast path
    if (a.n_plan) {
      const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(offsetof(GatherRuleArgs, plan))) + i);
      plan_kind = fp[7];
      plain = plan_kind == 0;
      to = reinterpret_cast<uint8_t *>(((uint64_t)fp[1] << 32 | fp[0]) + (uint64_t)r * fp[4]);
      to_a = to;
      len_a = fp[6];
      to_b = reinterpret_cast<uint8_t *>(((uint64_t)fp[3] << 32 | fp[2]) + (uint64_t)r * fp[5]);
    } else {
      plain = plain_target(a.app, 0, r, off, len, &to);
    }
  } else {
    to = dst + (uint64_t)r * size + off;
  }
  // offsets depend on the item, the size and the cursor only: they are out before a
  // fragment with a bad slot index is dropped
  if (slot >= n_slots) {
    if (lane == 0 && piece == 0) refuse(a.status, a.status_flag, kStBadSlot);
    return;
  }
  // The header words that hold the fragment's real length are fetched together
  // with the payload, so that checking them does not lengthen the wavefront's
  // life by another memory round trip.
  const bool check_hdr = piece == 0 && a.frag_len == nullptr;
  uint32_t hv = 0;
  u32x4 hc = {0u, 0u, 0u, 0u};
  if (check_hdr) {
    // every lane asks for the same bytes: one request, and on the cache line
    // the payload's first chunk needs anyway
    if (opts & kOptHdrChunk) hc = *reinterpret_cast<const u32x4 *>(pkt + 48);
    else hv = load32_any(pkt + 54);
  }
  // copying the ruled length stays inside the slot whatever the header says
  RunState rs;
  uint32_t sub_off = 0, sub_len = len;
  if (LONG && plain) sub_run(to, len, piece, &sub_off, &sub_len);
  if (plain && sub_len) run_begin(rs, pkt + hl + sub_off, to + sub_off, sub_len, lane);
  // a fragment that runs from one tensor into the next: two runs, both in flight at once
  const bool two = !plain && (opts & kOptMultiTensor) && piece == 0 &&
                   (plan_kind == 3 ? two_tensor_target(a.app, r, off, len, &to_a, &len_a, &to_b) : plan_kind == 1);
  RunState rb;
  // ... as ONE run with a break in its destination where the second tensor's share starts on a
  // 16-byte boundary and the first one's ends on a chunk boundary of the run (tensors of whole
  // chunks at aligned addresses)
  const uint32_t head_a = (uint32_t)(-(uintptr_t)to_a) & 15u;
  const bool one_run = two && ((uintptr_t)to_b & 15u) == 0 && len_a >= head_a && ((len_a - head_a) & 15u) == 0;
  if (one_run) {
    run_begin(rs, pkt + hl, to_a, len, lane);
  } else if (two) {
    run_begin(rs, pkt + hl, to_a, len_a, lane);
    run_begin(rb, pkt + hl + len_a, to_b, len - len_a, lane);
  }
  asm volatile("" ::"v"(hc), "v"(hv));  // consumed only after the payload loads are under way
  if (plain) {
    if (sub_len) run_end<false>(rs, lane);
  } else if (one_run) {
    run_end<false, true>(rs, lane, (len_a - head_a) >> 4, (int64_t)(to_b - (to_a + len_a)));
  } else if (two) {
    run_end<false>(rs, lane);
    run_end<false>(rb, lane);
  } else if (piece == 0) {
    move_run<true, false>(a.app, ro, r, off, pkt + hl, len, lane);
  }
  if (piece == 0) {
    uint32_t bad = 0;
    // payload_len is the u32 at byte 54: bytes 6..9 of the chunk that starts at byte 48
    const uint32_t hdr_len = (opts & kOptHdrChunk) ? ((hc[1] >> 16) | (hc[2] << 16)) : hv;
    const bool as_ruled = (check_hdr ? hdr_len : sload(a.frag_len + item)) == len;
    if (!as_ruled) bad |= kStNotRule;
    if (i == 0 && sload(a.first + r) != item) bad |= kStBadTable;
    if (bad && lane == 0) refuse(a.status, a.status_flag, bad);
  }
}

// Gather of SHORT fragments, 64 / L fragments per wavefront (L = 16 or 32 lanes
// per fragment): the rule form of the gather for fragments of a few hundred
// bytes -- every fragment of the call (per_launch == per_req) or the last
// fragment of every request (the remainder; the full fragments then go through
// k_gather_rule).  Addressing is per lane.
template <int L>
__device__ __forceinline__ void gather_small_wave(const GatherRuleArgs &a, uint32_t wave)
{
  constexpr uint32_t G = kWave / L;
  // every argument of the common path in one burst of scalar loads
  SG_PIN(a.per_req); SG_PIN(a.mtu); SG_PIN(a.hl); SG_PIN(a.counts); SG_PIN(a.n_req); SG_PIN(a.opts);
  SG_PIN(a.size); SG_PIN(a.frag_slot); SG_PIN(a.first); SG_PIN(a.n_slots); SG_PIN(a.cap); SG_PIN(a.cursor);
  SG_PIN(a.offsets_out); SG_PIN(a.ring); SG_PIN(a.slot_size); SG_PIN(a.frag_len); SG_PIN(a.dst);
  SG_PIN(a.n_plan); SG_PIN(a.div_mul); SG_PIN(a.div_shift);
  const uint32_t lane = threadIdx.x & (kWave - 1), gl = lane & (L - 1);
  const uint32_t per_req = a.per_req, mtu = a.mtu, hl = a.hl;
  const uint32_t n_req = dev_count(a.counts, 0, a.n_req);
  const bool last_only = (a.opts & kOptSmallLast) != 0;
  const uint32_t n_frags = last_only ? n_req : n_req * per_req;
  if (wave * G >= n_frags) return;  // the whole wavefront
  const uint32_t fi = wave * G + lane / L;
  bool live = fi < n_frags;
  uint32_t r = 0, i = 0, item = 0;
  if (live) {
    if (last_only) {
      r = fi;
      i = per_req - 1;
      item = r * per_req + i;
    } else {
      item = fi;
      r = (uint32_t)(((uint64_t)item * a.div_mul) >> a.div_shift);
      i = item - r * per_req;
    }
  }
  const uint32_t off = i * mtu;
  const uint32_t rem = (uint32_t)a.size - off;  // sizes are below 4 GiB (checked by the host)
  const uint32_t len = live ? (rem <= mtu ? rem : mtu) : 0u;
  const uint32_t slot = live ? a.frag_slot[item] : 0u;
  const uint32_t first_r = live && i == 0 ? a.first[r] : item;
  uint32_t bad = 0;
  if (slot >= a.n_slots) bad |= kStBadSlot;
  if (first_r != item) bad |= kStBadTable;
  // offsets depend on the item, the size and the cursor only: they are out before a bad fragment is dropped
  uint64_t ro = 0;
  if (a.cap) {
    uint64_t c0 = sload(a.cursor);
    if (c0 >= a.cap) c0 %= a.cap;  // only after a set_cursor beyond the capacity
    ro = c0 + (uint64_t)r * a.size;
    ro = ro >= a.cap ? ro - a.cap : ro;  // the batch fits the arena (checked by the host): one wrap at most
    if (live && gl == 0 && a.offsets_out) {
      if (i == 0) a.offsets_out[r] = ro;
      if (item == n_req * per_req - 1) {
        const uint64_t end = ro + a.size;  // size <= capacity
        a.offsets_out[n_req] = end >= a.cap ? end - a.cap : end;
      }
    }
  }
  if (live && (bad & kStBadSlot)) {
    if (gl == 0) refuse(a.status, a.status_flag, kStBadSlot);
    live = false;
  }
  const uint8_t *pkt = a.ring + (size_t)(live ? slot : 0u) * a.slot_size;
  // the fragment's real length, fetched with the payload
  uint32_t hdr_len = len;
  if (live && gl == 0) hdr_len = a.frag_len ? a.frag_len[item] : load32_any(pkt + 54);
  uint8_t *to = nullptr;
  bool plain = false;
  if (live && len) {
    if (a.cap) {
      // the packed arena, walked through the AppDev view the host filled in for this kernel
      plain = plain_target(a.app, ro, r, off, len, &to);
    } else if (a.opts & kOptMultiTensor) {
      if (last_only && a.n_plan) {
        // every group has the request's last fragment: one plan entry for the wavefront
        const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(offsetof(GatherRuleArgs, plan))) + (per_req - 1));
        plain = fp[7] == 0;
        to = reinterpret_cast<uint8_t *>(((uint64_t)fp[1] << 32 | fp[0]) + (uint64_t)r * fp[4]);
      } else {
        plain = plain_target(a.app, 0, r, off, len, &to);
      }
    } else {
      to = a.dst + (uint64_t)r * a.size + off;
      plain = true;
    }
  }
  GroupRun<L> run;
  group_run_begin<L>(run, pkt + hl, to, plain ? len : 0u, gl);
  group_run_end<L, false>(run, gl);
  if (live && len && !plain) {
    // across an arena end or a tensor boundary: byte by byte
    for (uint32_t k = gl; k < len; k += L) *app_byte(a.app, ro, r, (uint64_t)off + k) = pkt[hl + k];
  }
  if (live && gl == 0) {
    if (hdr_len != len) bad |= kStNotRule;
    if (bad) refuse(a.status, a.status_flag, bad);
  }
}

// Every fragment of the call is short.
template <int L>
__global__ __launch_bounds__(kBlock) void k_gather_small(GatherRuleArgs a)
{
  gather_small_wave<L>(a, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave);
}

struct ScatterArgs {
  const u32x4 *desc;
  const uint64_t *req_off;
  const uint32_t *first;         // resp_first CSR (for frag_idx / num_frags)
  const uint32_t *hdr_src_slot;
  const uint8_t *hdr_templates;  // non-null: headers from per-request templates, nothing swapped
  const uint64_t *req_token;
  const uint8_t *rx;
  uint32_t rx_slot_size;
  uint32_t rx_n_slots;
  uint8_t *tx;
  uint32_t tx_slot_size;
  uint32_t hl;
  uint32_t ref64;
  uint32_t flags;
  uint32_t n_items;
  uint32_t n_req;
  uint32_t remap;
  uint32_t pieces;  // wavefronts per frame
  uint32_t *status;
  volatile uint32_t *status_flag;  // pinned host word: non-zero once any kernel refused something
  uint64_t *cursor;             // descriptor path, packed: wavefront 0 commits *next_cursor
  const uint64_t *next_cursor;
  const uint32_t *hdr_src_req;  // one header source per request instead of hdr_src_slot per frame
  const uint32_t *counts;       // device-resident request count, or nullptr
  // full UDP checksum of long frames in two phases: every sub-run's wavefront leaves the sum of
  // its bytes in csum_part[frame * kPartStride + piece], wavefront 0 of a frame also the header's
  // share at [.. + pieces] and a mark in csum_valid[frame]; k_udp_finish folds them into the field
  uint32_t *csum_part;
  uint32_t *csum_valid;
  // SG_F_REUSE_DESC: the descriptors and offsets are those an earlier descriptor pass left (tagged
  // reuse_gen); they are held against the tag and the TX ring, and offsets_out is written from them
  const uint32_t *desc_tag;
  uint32_t reuse_gen;
  uint32_t tx_n_slots;
  uint64_t *offsets_out;
  RuleArgs rule;
  AppDev app;
  // fused, tensor-major buffers: where the bytes of frame i of a response come from (as
  // GatherRuleArgs::plan); n_plan == 0: the tensors are walked by the wavefront
  uint32_t n_plan;
  uint32_t plan_pad;
  FragPlan plan[kPlanMax];
};

// LONG: frames longer than kPieceChunks chunks are spread over a.pieces
// wavefronts; piece 0 also writes the header.  With the payload sum
// (FULL_CSUM) a long frame stays with one wavefront, which walks its sub-runs
// two at a time (more in flight cost registers, hence resident wavefronts, and
// measured slower: 3 at a time +1 %, 5 at a time +8 %).  (Summing per piece and combining with one returning atomic
// per wavefront was measured: the atomic's round trip at the end of every
// wavefront's life cost more than the shorter tail gained.)
// Where the payload of a frame comes from; false: not one contiguous piece.
template <bool FUSED>
__device__ __forceinline__ bool scatter_source(const ScatterArgs &a, uint64_t ro, uint32_t r, uint32_t i,
                                               uint32_t off, uint32_t len, uint8_t **from)
{
  if (FUSED && a.n_plan) {
    const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(offsetof(ScatterArgs, plan))) + i);
    *from = reinterpret_cast<uint8_t *>(((uint64_t)fp[1] << 32 | fp[0]) + (uint64_t)r * fp[4]);
    return fp[7] == 0;
  }
  return plain_target(a.app, ro, r, off, len, from);
}

constexpr uint32_t kPartStride = 8;  // words of csum_part per frame: up to 7 sub-runs and the header's share

// DEFER (long frames with the full UDP checksum): the frame's sub-runs go to
// several wavefronts all the same, each leaving the sum of its bytes behind,
// and k_udp_finish writes the checksum field afterwards.
template <bool FULL_CSUM, bool FUSED, bool LONG, bool DEFER = false>
__global__ __launch_bounds__(kBlock) void k_scatter(ScatterArgs a)
{
  constexpr bool SPLIT = LONG && (!FULL_CSUM || DEFER);      // several wavefronts per frame
  constexpr bool WHOLE_LONG = LONG && FULL_CSUM && !DEFER;   // one wavefront walks all sub-runs of its frame
  // every argument of the common path in one burst of scalar loads
  const u32x4 *desc = a.desc;
  const uint64_t *req_off = a.req_off;
  const uint32_t *first = a.first, *hdr_src_slot = a.hdr_src_slot;
  const uint8_t *hdr_templates = a.hdr_templates, *rx = a.rx;
  uint8_t *tx = a.tx;
  const uint32_t rx_slot_size = a.rx_slot_size, rx_n_slots = a.rx_n_slots, tx_slot_size = a.tx_slot_size;
  const uint32_t hl = a.hl, remap = a.remap, n_pieces = a.pieces;
  const uint32_t *status = a.status;
  const uint32_t *counts = a.counts, *hdr_src_req = a.hdr_src_req;
  uint32_t n_items = a.n_items, n_req = a.n_req;
  SG_PIN(desc); SG_PIN(req_off); SG_PIN(first); SG_PIN(hdr_src_slot); SG_PIN(hdr_templates); SG_PIN(rx);
  SG_PIN(tx); SG_PIN(rx_slot_size); SG_PIN(rx_n_slots); SG_PIN(tx_slot_size); SG_PIN(hl); SG_PIN(n_items);
  SG_PIN(remap); SG_PIN(n_pieces); SG_PIN(status); SG_PIN(counts); SG_PIN(hdr_src_req);
  if (counts) {
    // the launch was sized for n_req responses at most; the frame table ends where the live ones end
    n_req = dev_count(counts, 0, n_req);
    const uint32_t live = FUSED ? n_req * a.rule.per_req : (n_req ? sload(first + n_req) : 0u);
    n_items = live < n_items ? live : n_items;
  }
  SG_PIN(a.app.n_tensors); SG_PIN(a.app.arena); SG_PIN(a.app.cap); SG_PIN(a.app.mirrored);
  if (FUSED) {
    SG_PIN(a.rule.item_slot); SG_PIN(a.rule.first); SG_PIN(a.rule.size); SG_PIN(a.rule.mtu);
    SG_PIN(a.rule.per_req); SG_PIN(a.rule.n_slots); SG_PIN(a.rule.single_wrap); SG_PIN(a.rule.cursor);
  }
  const uint32_t w = item_of_wave(remap != 0);
  const uint32_t pieces = SPLIT ? n_pieces : 1u;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  // descriptor path: this kernel does not read the cursor and commits what the descriptor pass left
  if (!FUSED && a.reuse_gen && n_req) {
    // the caller says these are the items the tagged descriptor pass described
    if (sload(a.desc_tag) != a.reuse_gen || sload(a.desc_tag + 1) != n_req || sload(a.desc_tag + 2) != n_items) {
      if (w == 0 && lane == 0) refuse(a.status, a.status_flag, kStBadTable);
      return;
    }
  }
  if (!FUSED && w == 0 && lane == 0 && a.cursor && !sload(status) && (!counts || sload(counts))) {
    const uint64_t nc = sload(a.next_cursor);
    *a.cursor = nc;
    if (a.reuse_gen && a.offsets_out) a.offsets_out[n_req] = nc;
  }
  uint32_t item = SPLIT ? w / pieces : w;
  const uint32_t piece = SPLIT ? w - item * pieces : 0;
  if (FUSED && a.rule.per_launch != a.rule.per_req) {
    // the short remainder frame of every response is k_scatter_small's (a launch of its own: with
    // both kinds of wavefront in one kernel, in turns or one kind after the other, the full frames
    // lost more than the second launch costs): this launch counts the other frames only
    const uint32_t pl = a.rule.per_launch;
    if (item >= n_req * pl) return;
    const uint32_t rr = (uint32_t)(((uint64_t)item * a.rule.lmul) >> a.rule.lshift);
    item = rr * a.rule.per_req + (item - rr * pl);
  }
  if (item >= n_items) return;
  const bool from_template = hdr_templates != nullptr;
  // independent table reads, asked for together
  uint32_t hs = (from_template || hdr_src_req) ? 0u : sload_here(hdr_src_slot + item);
  u32x4 d;
  uint32_t r, f0, nf;
  uint64_t ro;
  if (!FUSED) {
    d = sload_here(desc + item);
    if (sload_here(status)) return;  // the descriptor pass refused the batch: move nothing
    r = d[3];
    if (r == kInvalidReq) return;
    f0 = sload(first + r);
    nf = sload(first + r + 1) - f0;
    ro = a.app.n_tensors == 0 ? sload(req_off + r) : 0;
    if (a.reuse_gen) {
      if (d[0] >= a.tx_n_slots) {  // described for another ring
        if (lane == 0 && piece == 0) refuse(a.status, a.status_flag, kStBadSlot);
        return;
      }
      if (a.offsets_out && item == f0 && lane == 0 && piece == 0) a.offsets_out[r] = ro;
    }
  } else {
    uint32_t slot_i, len, off, i;
    const uint32_t bad = rule_desc(a.rule, a.app, item, n_items, n_req, piece == 0 ? lane : 1u, &slot_i, &len,
                                   &off, &r, &i, &ro);
    if (bad) {
      if (lane == 0 && piece == 0) refuse(a.status, a.status_flag, bad);
      return;
    }
    d = (u32x4){slot_i, len, off, r};
    f0 = item - i;
    nf = a.rule.per_req;
  }
  uint8_t *slot = tx + (size_t)d[0] * tx_slot_size;
  // where the header comes from; a frame whose header source is out of range is left alone by
  // all of its pieces
  const uint8_t *hin;
  HdrFields hf{hl, a.ref64, a.flags, item - f0, nf, d[1], 0, 0, 0};
  if (from_template) {
    hin = hdr_templates + (size_t)r * 64;
    hf.from_template = 1;
    if (a.req_token) {
      hf.set_token = 1;
      hf.token = a.req_token[r];
    }
  } else {
    if (hdr_src_req) hs = sload(hdr_src_req + r);
    if (hs >= rx_n_slots) {
      // descriptor path: the descriptor pass has refused the batch already and nothing gets here
      // (unless its descriptors are being reused: no pass has seen this call's header sources)
      if ((FUSED || a.reuse_gen) && lane == 0 && piece == 0) refuse(a.status, a.status_flag, kStBadSlot);
      return;
    }
    hin = rx + (size_t)hs * rx_slot_size;
  }

  if (SPLIT && piece != 0) {
    // a later piece of a long frame: payload only
    uint8_t *from;
    uint32_t part = 0;
    if (d[1] && scatter_source<FUSED>(a, ro, r, item - f0, d[2], d[1], &from)) {
      uint32_t o, n;
      sub_run(slot + hl, d[1], piece, &o, &n);
      if (n) part = copy_run<DEFER>(from + o, slot + hl + o, n, lane);
    }
    if (DEFER) {
      part = wave_sum_uniform(part);
      if (lane == 0) a.csum_part[(size_t)item * kPartStride + piece] = part;
    }
    return;
  }
  // read the request header before anything of this slot is overwritten
  // (the TX slot may be the very slot the header comes from);
  // header bytes and payload chunks are fetched together; the header arithmetic
  // then runs while the payload is still on its way
  const uint32_t raw = hdrw_fetch(hin, lane, hl, !from_template);
  uint32_t hb = 0, acc = 0;
  uint8_t *from = nullptr;
  const bool plain = d[1] != 0 && scatter_source<FUSED>(a, ro, r, item - f0, d[2], d[1], &from);
  RunState rs;
  uint32_t first_len = d[1];
  if (SPLIT && plain) {
    uint32_t o;
    sub_run(slot + hl, d[1], 0, &o, &first_len);
  }
  if (plain && !WHOLE_LONG) run_begin(rs, from, slot + hl, first_len, lane);
  hb = hdrw_fields(raw, hf);
  if (!FULL_CSUM) hb = hdrw_csums(hb, hf, 0);
  if (plain) {
    if (WHOLE_LONG) acc = copy_long_run<FULL_CSUM, 2>(from, slot + hl, d[1], lane);
    else acc = run_end<FULL_CSUM>(rs, lane);
  } else if (d[1]) {
    acc = move_run<false, FULL_CSUM>(a.app, ro, r, d[2], slot + hl, d[1], lane);
  }
  // the header's own share of the UDP sum rides with the payload's
  if (FULL_CSUM) acc += hdrw_l4_share(hb, lane, hl);
  if (FULL_CSUM && !DEFER) hb = hdrw_csums(hb, hf, wave_sum_uniform(acc));
  if (DEFER) {
    uint32_t l4 = 0;
    hb = hdrw_csums(hb, hf, 0, &l4);
    const uint32_t part = wave_sum_uniform(acc);
    if (lane == 0) {
      a.csum_part[(size_t)item * kPartStride] = part;
      a.csum_part[(size_t)item * kPartStride + n_pieces] = l4;
      a.csum_valid[item] = 1u;  // this frame was written: its checksum field is to be finished
    }
  }
  // the payload went past the header only, so a TX slot that is the header's own
  // source still held the request header when it was fetched above
  hdrw_store(slot, lane, hl, hb);
}

// Second phase of the full UDP checksum of long frames: one thread per frame
// folds the sums its wavefronts left and writes the field (bytes 40, 41).
// Frames that were not written (refused) carry no mark and are left alone;
// marks are taken down for the next call.
template <bool FUSED>
__global__ __launch_bounds__(kBlock) void k_udp_finish(ScatterArgs a)
{
  const uint32_t item = blockIdx.x * kBlock + threadIdx.x;
  uint32_t n_items = a.n_items;
  if (a.counts) {
    const uint32_t n_req = dev_count(a.counts, 0, a.n_req);
    const uint32_t live = FUSED ? n_req * a.rule.per_req : (n_req ? a.first[n_req] : 0u);
    n_items = live < n_items ? live : n_items;
  }
  if (item >= n_items) return;
  // everything this thread reads, asked for at once: the mark, the frame's eight words, its slot
  const u32x4 *p = reinterpret_cast<const u32x4 *>(a.csum_part + (size_t)item * kPartStride);
  const uint32_t valid = a.csum_valid[item];
  const u32x4 lo = p[0], hi = p[1];
  const uint32_t slot = FUSED ? a.rule.item_slot[item] : a.desc[item][0];
  if (!valid) return;
  a.csum_valid[item] = 0;
  const uint32_t w[kPartStride] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  uint32_t sum = 0, hdr = 0;
#pragma unroll
  for (uint32_t k = 0; k < kPartStride; k++) {
    if (k < a.pieces) sum += w[k];  // each below 2^27
    if (k == a.pieces) hdr = w[k];
  }
  uint32_t s = fold16(fold16(hdr) + fold16(sum));
  uint32_t c = (~s) & 0xffffu;
  if (c == 0) c = 0xffffu;
  // slots start at even addresses; the sums ran over the words as they lie in memory
  *reinterpret_cast<uint16_t *>(a.tx + (size_t)slot * a.tx_slot_size + 40) = (uint16_t)c;
}

// Scatter of SHORT frames, 64 / L frames per wavefront (L = 16 or 32 lanes per
// frame): the fused form of k_scatter -- responses of one size cut by the
// fragmenting rule -- for frames of a few hundred bytes, where one wavefront per
// frame spends most of its time on addressing and header arithmetic that 48 of
// its 64 lanes take no part in.  Either every frame of the call (rule.per_launch
// == rule.per_req) or the last frame of every response (the remainder; the full
// frames then go through k_scatter).  Addressing is per lane, the header is two
// 16-bit words per lane, sums are row reductions.
template <int L, bool FULL_CSUM>
__device__ __forceinline__ void scatter_small_wave(const ScatterArgs &a, uint32_t wave)
{
  constexpr uint32_t G = kWave / L;
  // every argument of the common path in one burst of scalar loads (left to their first uses they
  // arrive one dependent round trip after the other, a good part of this wavefront's life)
  SG_PIN(a.rule.per_req); SG_PIN(a.rule.mtu); SG_PIN(a.hl); SG_PIN(a.counts); SG_PIN(a.n_req);
  SG_PIN(a.rule.per_launch); SG_PIN(a.rule.size); SG_PIN(a.hdr_templates); SG_PIN(a.rule.item_slot);
  SG_PIN(a.rule.first); SG_PIN(a.hdr_src_req); SG_PIN(a.hdr_src_slot); SG_PIN(a.rule.n_slots);
  SG_PIN(a.rx_n_slots); SG_PIN(a.app.n_tensors); SG_PIN(a.rule.cursor); SG_PIN(a.app.cap);
  SG_PIN(a.rule.single_wrap); SG_PIN(a.rule.offsets_out); SG_PIN(a.rule.div_mul); SG_PIN(a.rule.div_shift);
  SG_PIN(a.req_token); SG_PIN(a.rx); SG_PIN(a.rx_slot_size); SG_PIN(a.tx); SG_PIN(a.tx_slot_size);
  SG_PIN(a.ref64); SG_PIN(a.flags); SG_PIN(a.n_plan); SG_PIN(a.app.arena); SG_PIN(a.app.mirrored);
  const uint32_t lane = threadIdx.x & (kWave - 1), gl = lane & (L - 1);
  const uint32_t per_req = a.rule.per_req, mtu = a.rule.mtu, hl = a.hl;
  const uint32_t n_req = dev_count(a.counts, 0, a.n_req);
  const bool last_only = a.rule.per_launch != per_req;
  const uint32_t n_frames = last_only ? n_req : n_req * per_req;
  if (wave * G >= n_frames) return;  // the whole wavefront
  const uint32_t fi = wave * G + lane / L;
  bool live = fi < n_frames;
  uint32_t r = 0, i = 0, item = 0;
  if (live) {
    if (last_only) {
      r = fi;
      i = per_req - 1;
      item = r * per_req + i;
    } else {
      item = fi;
      r = (uint32_t)(((uint64_t)item * a.rule.div_mul) >> a.rule.div_shift);
      i = item - r * per_req;
    }
  }
  const uint32_t off = i * mtu;
  const uint32_t rem = (uint32_t)a.rule.size - off;  // response sizes are below 4 GiB (checked by the host)
  const uint32_t len = live ? (rem <= mtu ? rem : mtu) : 0u;
  const bool from_template = a.hdr_templates != nullptr;
  // tables: independent reads
  uint32_t bad = 0;
  const uint32_t tslot = live ? a.rule.item_slot[item] : 0u;
  const uint32_t first_r = live ? a.rule.first[r] : 0u;
  uint32_t hs = 0;
  if (live && !from_template) hs = a.hdr_src_req ? a.hdr_src_req[r] : a.hdr_src_slot[item];
  // Where the payload comes from depends on the frame's number alone, and so does the phase of
  // where it goes when slots lie whole chunks apart: its loads are asked for now, a round trip
  // before the tables above say which slot the frame goes to (and whether it goes at all).
  const bool early = (a.tx_slot_size & 15u) == 0;
  uint64_t ro = 0;
  if (a.app.n_tensors == 0) {
    uint64_t c0 = sload(a.rule.cursor);
    if (c0 >= a.app.cap) c0 %= a.app.cap;  // only after a set_cursor beyond the capacity
    uint64_t o = c0 + (uint64_t)r * a.rule.size;
    if (a.rule.single_wrap) o = o >= a.app.cap ? o - a.app.cap : o;
    else o %= a.app.cap;
    ro = o;
  }
  uint8_t *from = nullptr;
  bool plain;
  if (last_only && a.n_plan) {
    // every group has the response's last frame: one plan entry for the wavefront
    const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(offsetof(ScatterArgs, plan))) + (per_req - 1));
    from = reinterpret_cast<uint8_t *>(((uint64_t)fp[1] << 32 | fp[0]) + (uint64_t)r * fp[4]);
    plain = live && len != 0 && fp[7] == 0;
  } else {
    plain = live && len != 0 && plain_target(a.app, ro, r, off, len, &from);
  }
  GroupRun<L> run;
  if (early)
    group_run_begin<L>(run, from, reinterpret_cast<uint8_t *>(((uintptr_t)a.tx + hl) & 15u), plain ? len : 0u, gl);
  if (tslot >= a.rule.n_slots) bad |= kStBadSlot;
  if (i == 0 && first_r != item) bad |= kStBadTable;
  if (hs >= a.rx_n_slots) bad |= kStBadSlot;
  if (live && bad && gl == 0) refuse(a.status, a.status_flag, bad);
  // offsets depend on the item, the size and the cursor only: they are out before a bad frame is dropped
  if (a.app.n_tensors == 0 && live && gl == 0 && a.rule.offsets_out) {
    if (i == 0) a.rule.offsets_out[r] = ro;
    if (item == n_req * per_req - 1) {
      const uint64_t end = ro + a.rule.size;  // size <= capacity
      a.rule.offsets_out[n_req] = end >= a.app.cap ? end - a.app.cap : end;
    }
  }
  live = live && !bad;
  plain = plain && live;
  uint8_t *slot = a.tx + (size_t)tslot * a.tx_slot_size;
  HdrFields hf{hl, a.ref64, a.flags, i, per_req, len, 0, 0, 0};
  const uint8_t *hin;
  if (from_template) {
    hin = a.hdr_templates + (size_t)r * 64;
    hf.from_template = 1;
    if (a.req_token) {
      hf.set_token = 1;
      hf.token = live ? a.req_token[r] : 0;
    }
  } else {
    hin = a.rx + (size_t)hs * a.rx_slot_size;
  }
  // header words and payload chunks are fetched together; a TX slot that is its own header
  // source still holds the request header then (the payload goes past the header only)
  const SmallHdr sh = small_hdr_fetch(hin, gl, hl, !from_template, live && gl < 16);
  if (early) {
    group_run_rebase<L>(run, slot + hl);
    if (!plain) group_run_cancel<L>(run);  // a frame the tables have just ruled out
  } else {
    group_run_begin<L>(run, from, slot + hl, plain ? len : 0u, gl);
  }
  uint32_t acc = group_run_end<L, FULL_CSUM>(run, gl);
  if (live && len != 0 && !plain) {
    // across an arena end or a tensor boundary: byte by byte
    for (uint32_t k = gl; k < len; k += L) {
      const uint32_t b = *app_byte(a.app, ro, r, (uint64_t)off + k);
      slot[hl + k] = (uint8_t)b;
      if (FULL_CSUM) acc += ((uintptr_t)(slot + hl + k) & 1u) ? (b << 8) : b;
    }
  }
  const uint32_t psum = FULL_CSUM ? group_sum<L>(acc) : 0u;
  small_hdr_finish<L>(sh, slot, gl, hf, psum, live);
}

// Every frame of the call is short.
template <int L, bool FULL_CSUM>
__global__ __launch_bounds__(kBlock) void k_scatter_small(ScatterArgs a)
{
  scatter_small_wave<L, FULL_CSUM>(a, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave);
}

// ---------------------------------------------------------------------------
// per-request entry points
// ---------------------------------------------------------------------------

struct Run {
  uint64_t src;
  uint64_t dst;
  uint64_t len;
};

__global__ __launch_bounds__(kBlock) void k_copy_runs(const Run *runs, uint32_t n)
{
  const uint32_t item = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (item >= n) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const Run r = runs[item];
  copy_run<false>(reinterpret_cast<const uint8_t *>(r.src), reinterpret_cast<uint8_t *>(r.dst),
                  (uint32_t)r.len, lane);
}

// tmpl == nullptr: swap each header in place; else every header is a copy of
// the 64-byte template with `token` in it (the two ways the reference fills
// response headers: rr_swap_hdr and rr_set_hdr).
__global__ __launch_bounds__(kBlock) void k_swap_hdrs(const uint64_t *hdr_ptrs, uint32_t n,
                                                      uint32_t hl, uint32_t ref64, uint32_t flags,
                                                      uint64_t payload_size, uint32_t mtu,
                                                      const uint8_t *tmpl, uint64_t token)
{
  const uint32_t item = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (item >= n) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint8_t *h = reinterpret_cast<uint8_t *>(hdr_ptrs[item]);
  const uint64_t taken = (uint64_t)item * mtu;
  const uint64_t rem = taken < payload_size ? payload_size - taken : 0;
  HdrFields hf{hl, ref64, flags & ~(1u << 2), item, n, (uint32_t)(rem <= mtu ? rem : mtu),
               tmpl != nullptr, tmpl != nullptr, token};
  const uint32_t b = hdr_finish(hdr_fetch(tmpl ? tmpl : h, lane, hl, tmpl == nullptr), lane, hf, 0);
  if (lane < hl) h[lane] = (uint8_t)b;
}

// ---------------------------------------------------------------------------
// request reassembly on the device
// ---------------------------------------------------------------------------
// What the receive thread of the reference does per packet -- look the request
// up by token (get_rr), file the fragment at its sequence number
// (rr_emplace_mbuf), hand the request over once complete (is_rr_ready,
// mark_rx_ready_rr) -- done for a whole burst of arrivals at once, with the
// requests that are still incomplete kept on the device from call to call, as
// rr_cache keeps them (src/p2p_rpc_rr_pool_ng.h:97-119):
//   request table   token -> cell, open addressing in buckets of kRaBucket
//                   cells: a lookup reads the whole bucket, so emptying a cell
//                   (a completed request) never hides another request, and a
//                   new token claims the lowest empty cell by atomicCAS
//   record pool     one record per request in flight: SG_MAX_BI_SIZE entries
//                   {slot, length} indexed by sequence number (p2p_bufs of the
//                   reference's rr); free records wait in a ring with a head
//                   and a tail word on the device (the rr pool's free ring,
//                   src/p2p_rpc_rr_pool_ng.h:121-147: consume_rr / reap_rr)
//   k_ra_insert  one thread per arrival: find or claim the request's cell (a
//                claimed cell takes a record off the free ring), add to its
//                fragment count / byte total, note the arrival's position
//   k_ra_flag    every arrival files its entry in its request's record; the
//                thread of a complete request's LAST arrival flags that
//                position with the request's fragment count; workgroup-local
//                scan of the packed (requests, fragments) flags
//   k_ra_scan    one workgroup scans the workgroup totals and leaves the counts
//                on the device and in pinned host memory
//   k_ra_emit    batch index of a request = number of requests completed before
//                it in this call (completion order, the order of the rx-ready
//                ring); the wavefront of the completing arrival copies the
//                record into the output tables, empties it, returns it to the
//                free ring and empties the cell
// Nothing waits on another thread: every probe and every ring operation makes
// progress by itself.

constexpr uint32_t kRaBucket = 32;
static_assert(kRaBucket == 32, "ra_find_cell takes a token's first cell from the top five bits of its hash");
constexpr uint32_t kRaNoCell = 0xffffffffu;
constexpr uint32_t kRaNoRec = 0xffffffffu;
constexpr int kRaBlock = 1024;
// device words of the reassembly state
// kRaHeadSeen: where k_ra_scan last saw the head -- how far it has moved since is the number of
// cells claimed in between
enum { kRaHead = 0, kRaTail, kRaEpoch, kRaInFlight, kRaHeadSeen, kRaDropped, kRaOverflow, kRaEvicted, kRaWords = 16 };

struct RaArgs {
  const uint8_t *ring;
  uint32_t n_slots, slot_size, ref64;
  uint32_t n;             // arrivals of this call, or their upper bound with n_dev
  const uint32_t *n_dev;  // device-resident arrival count, or nullptr
  const uint32_t *arrivals;
  const uint32_t *len_nic;
  uint64_t req_size;  // REF64 readiness: bytes == req_size; BL58: fragments == num_frags
  uint32_t bmask;     // buckets - 1
  uint32_t rmask;     // records - 1
  uint32_t max_req, max_frag;  // room in the output tables
  // request table: cells
  unsigned long long *keys;
  unsigned long long *acc;  // fragments so far << 40 | payload bytes so far: one atomic addition per arrival
  uint32_t *want, *last, *rec, *seen;
  // record pool
  unsigned long long *tab;  // records x SG_MAX_BI_SIZE entries: slot | length << 32
  uint32_t *free_ring;
  uint32_t *words;          // kRa* above
  // per arrival of this call
  uint32_t *arr_cell, *arr_len, *arr_fidx;
  unsigned long long *arr_pack;  // (1 << 32 | fragments) at the completing arrival, else 0; then its local scan
  unsigned long long *blk;       // workgroup totals, then their scan
  uint32_t n_blocks;
  // outputs
  uint32_t *frag_slot, *frag_len, *req_first, *req_hdr_slot;
  uint64_t *req_token;
  uint32_t *counts_out;            // device: requests, fragments, arrivals dropped, requests in flight
  volatile uint32_t *counts_host;  // the same four, pinned host memory
  uint32_t *status;
  volatile uint32_t *status_flag;  // pinned host word: non-zero once any kernel refused something
};

__device__ __forceinline__ uint32_t ra_n(const RaArgs &a)
{
  return dev_count(a.n_dev, 0, a.n);
}

// A cell's fragment count and byte total in one word (a request has at most SG_MAX_BI_SIZE
// fragments and far fewer than 2^40 bytes): device-scope atomics are what a burst of many small
// requests pays for, one per arrival instead of two.
constexpr int kRaCntShift = 40;
__device__ __forceinline__ unsigned long long ra_pack(uint32_t n, unsigned long long bytes)
{
  return ((unsigned long long)n << kRaCntShift) + bytes;
}
__device__ __forceinline__ uint32_t ra_cnt(unsigned long long acc) { return (uint32_t)(acc >> kRaCntShift); }
__device__ __forceinline__ unsigned long long ra_bytes(unsigned long long acc)
{
  return acc & ((1ull << kRaCntShift) - 1ull);
}

__device__ __forceinline__ uint32_t ra_hash(unsigned long long k)
{
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  return (uint32_t)k;
}

__device__ __forceinline__ unsigned long long ra_key(const unsigned long long *p)
{
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Find or claim the cell of `token`.  The whole bucket is read first: the
// request may sit anywhere in it (cells empty as requests complete).  Only then
// is an empty cell claimed.  Every token walks the bucket in an order of its
// own -- cyclically from a cell its hash picks -- starting at the first cell of
// that order it has seen empty and trying every empty cell on the way; cells
// before that one in the order were taken when they were read and stay taken
// while arrivals are being filed, so two threads that bring the same new token
// end up in the same cell whatever else is claimed around them.  (With one
// order for all tokens -- lowest cell first -- the new requests of a burst that
// share a bucket queued up on its lowest empty cells, one failed
// compare-and-swap round trip after the other.)
__device__ __forceinline__ uint32_t ra_find_cell(const RaArgs &a, unsigned long long token, bool *claimed)
{
  const uint32_t hash = ra_hash(token);
  const uint32_t b = (hash & a.bmask) * kRaBucket;
  const uint32_t start = hash >> 27;  // kRaBucket == 32: the top five bits, the bucket takes the low ones
  *claimed = false;
  uint32_t first_rank = kRaBucket;  // place in this token's order of the first cell seen empty
#pragma unroll 1
  for (uint32_t h = 0; h < kRaBucket; h += 16) {
    // Ordinary 16-byte loads, two keys each.  While arrivals are being filed a key only ever goes
    // from empty to a token, so all a load that is behind the times can show is an empty cell that
    // has just been taken -- and the claim below goes through atomicCAS, which then returns the
    // taker (this thread's own token included).
    unsigned long long k[16];
    const ulonglong2 *kp = reinterpret_cast<const ulonglong2 *>(a.keys + b + h);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const ulonglong2 v = kp[j];
      k[2 * j] = v.x;
      k[2 * j + 1] = v.y;
    }
#pragma unroll
    for (int j = 0; j < 16; j++) {
      if (k[j] == token) return b + h + j;
      const uint32_t rank = (h + j - start) & (kRaBucket - 1);
      if (k[j] == 0ull && rank < first_rank) first_rank = rank;
    }
  }
#pragma unroll 1
  for (uint32_t rank = first_rank; rank < kRaBucket; rank++) {
    const uint32_t j = (start + rank) & (kRaBucket - 1);
    unsigned long long k = rank == first_rank ? 0ull : ra_key(a.keys + b + j);
    if (k == 0ull) {
      k = atomicCAS(&a.keys[b + j], 0ull, token);
      if (k == 0ull) {
        *claimed = true;
        return b + j;
      }
    }
    if (k == token) return b + j;
  }
  return kRaNoCell;  // bucket full
}

// Positions on a ring word for a whole workgroup with ONE addition: every wavefront says how many it
// needs and gets its first.  (A returning addition per wavefront on a word that thousands of wavefronts
// on eight XCDs add to takes some 70 ns, one after the other: 0.29 ms of a 0.35-ms k_ra_insert on a
// burst of 131072 new requests.)  Every thread of the workgroup has to call this.
constexpr int kRaTakeBlock = 1024;
__device__ __forceinline__ uint32_t ra_block_take(uint32_t *word, uint32_t n_wave, uint32_t *lds)
{
  constexpr uint32_t kWaves = kRaTakeBlock / kWave;
  const uint32_t wv = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wv] = n_wave;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t tot = 0;
    for (uint32_t w = 0; w < kWaves; w++) {
      const uint32_t t = lds[w];
      lds[w] = tot;
      tot += t;
    }
    lds[kWaves] = tot ? atomicAdd(word, tot) : 0u;
  }
  __syncthreads();
  return lds[kWaves] + lds[wv];
}

// Records for the cells the threads of this workgroup have just claimed: one addition to the
// ring's head for all of them.  The tail does not move during the kernel that takes records
// (returns happen in k_ra_emit), so a position at or beyond the tail read here means the pool is
// exhausted: the cell then gets no record, the call is refused, and k_ra_scan puts the head back
// to the tail.
__device__ __forceinline__ void ra_open_cells(const RaArgs &a, bool claimed, uint32_t cell, uint32_t lane, uint32_t *lds)
{
  const unsigned long long cl = __ballot(claimed);
  const uint32_t base = ra_block_take(&a.words[kRaHead], (uint32_t)__popcll(cl), lds);
  if (claimed) {
    const uint32_t h = base + (uint32_t)__popcll(cl & ((1ull << lane) - 1ull));
    const uint32_t tail = a.words[kRaTail];
    const uint32_t r = (int32_t)(tail - h) > 0 ? a.free_ring[h & a.rmask] : kRaNoRec;
    a.rec[cell] = r;
    if (r == kRaNoRec) refuse(a.status, a.status_flag, kStPoolFull);
  }
}

// Fragments of one request tend to arrive together, so the lanes of a
// wavefront are first grouped by token: a group's first lane looks the cell up
// once and adds the group's fragment count, bytes and last position in one
// atomic each.  After kRaRounds groups the lanes still waiting go one by one
// (bursts that interleave many requests).
constexpr int kRaRounds = 4;

// The four steps of a call as functions of the arrival's index: launched as four kernels, or --
// a burst that fits one workgroup, which is what a NIC delivers -- one behind the other in ONE
// kernel (FUSED), with workgroup barriers where the kernel boundaries were.  What a step reads of
// what other threads left through device-scope atomics in an earlier step of the same kernel
// (counts and bytes, last positions, keys, ring words) it then reads with device-scope loads: an
// ordinary load could still find the line as a cache held it before the atomic went to memory.
template <bool FUSED>
__device__ __forceinline__ unsigned long long ra_acc(const RaArgs &a, uint32_t cell)
{
  return FUSED ? __hip_atomic_load(a.acc + cell, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : a.acc[cell];
}
template <bool FUSED>
__device__ __forceinline__ uint32_t ra_word(const uint32_t *p)
{
  return FUSED ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
}

__device__ __forceinline__ void ra_insert_step(const RaArgs &a, uint32_t i, uint32_t *take)
{
  const uint32_t n = ra_n(a);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const bool in_range = i < n;
  const uint32_t epoch = a.words[kRaEpoch];  // advanced by k_ra_scan, behind this kernel
  uint32_t cell = kRaNoCell, len = 0, fidx = 0, want = 0;
  uint32_t opened = kRaNoCell;  // the cell this lane has claimed for a new request, if any
  unsigned long long token = 0;
  bool pending = false;
  if (in_range) {
    const uint32_t slot = a.arrivals[i];
    if (slot >= a.n_slots) {
      refuse(a.status, a.status_flag, kStBadSlot);
    } else {
      const uint8_t *h = a.ring + (size_t)slot * a.slot_size;
      const uint32_t t0 = load32_any(h + 42), t1 = load32_any(h + 46);
      token = ((unsigned long long)t1 << 32) | t0;
      if (a.ref64) {
        fidx = load32_any(h + 58) & 0xffffu;
        len = a.len_nic[slot];
      } else {
        const uint32_t w = load32_any(h + 50);
        fidx = w & 0xffffu;
        want = w >> 16;
        len = a.len_nic ? a.len_nic[slot] : load32_any(h + 54);
      }
      const uint32_t hl = a.ref64 ? 64u : 58u;
      if (len > a.slot_size - hl) {
        refuse(a.status, a.status_flag, kStBadLen);
        len = 0;
      } else {
        pending = token != 0;  // token 0: dropped (src/transport/dpdk_transport_ng.h:231)
      }
    }
  }
  for (int round = 0; round < kRaRounds; round++) {
    const unsigned long long waiting = __ballot(pending);
    if (!waiting) break;
    const int first = __ffsll((long long)waiting) - 1;
    const unsigned long long t = ((unsigned long long)(uint32_t)__shfl((int)(token >> 32), first, kWave) << 32) |
                                 (uint32_t)__shfl((int)(uint32_t)token, first, kWave);
    const bool mine = pending && token == t;
    const unsigned long long group = __ballot(mine);
    // a burst that interleaves many requests: groups of one or two lanes, each a chain of
    // dependent round trips that the other lanes sit out -- every lane for itself then
    if (round == 0 && 8 * __popcll(group) < __popcll(waiting)) break;
    const uint32_t g_bytes = wave_sum(mine ? len : 0u);
    uint32_t c = kRaNoCell;
    if ((int)lane == first) {
      bool claimed;
      c = ra_find_cell(a, t, &claimed);
      if (c != kRaNoCell) {
        if (claimed) opened = c;
        atomicAdd(&a.acc[c], ra_pack((uint32_t)__popcll(group), g_bytes));
        atomicMax(&a.last[c], i - lane + (63u - (uint32_t)__clzll((long long)group)));
        if (!a.ref64) a.want[c] = want;  // every fragment of a request says the same
        a.seen[c] = epoch;
      }
    }
    c = (uint32_t)__shfl((int)c, first, kWave);
    if (mine) {
      cell = c;
      pending = false;
    }
  }
  if (pending) {
    bool claimed;
    cell = ra_find_cell(a, token, &claimed);
    if (cell != kRaNoCell) {
      if (claimed) opened = cell;
      atomicAdd(&a.acc[cell], ra_pack(1u, len));
      atomicMax(&a.last[cell], i);
      if (!a.ref64) a.want[cell] = want;
      a.seen[cell] = epoch;
    }
  }
  // the cells this wavefront has claimed get their records (a lane claims one cell at most)
  ra_open_cells(a, opened != kRaNoCell, opened, lane, take);
  if (in_range) {
    a.arr_cell[i] = cell;
    a.arr_len[i] = len;
    a.arr_fidx[i] = fidx;
    if (cell == kRaNoCell && token != 0) refuse(a.status, a.status_flag, kStPoolFull);  // bucket full
  }
  // arrivals that belong to no request: token 0, refused, no room
  const unsigned long long lost = __ballot(in_range && cell == kRaNoCell);
  if (lane == 0 && lost) atomicAdd(&a.words[kRaDropped], (uint32_t)__popcll(lost));
}

__global__ __launch_bounds__(kRaTakeBlock) void k_ra_insert(RaArgs a)
{
  __shared__ uint32_t take[kRaTakeBlock / kWave + 1];
  ra_insert_step(a, blockIdx.x * kRaTakeBlock + threadIdx.x, take);
}

__device__ __forceinline__ bool ra_complete(const RaArgs &a, uint32_t cell, unsigned long long acc)
{
  return a.ref64 ? ra_bytes(acc) == a.req_size : ra_cnt(acc) == a.want[cell];
}

// Returns the workgroup's packed (requests, fragments) total.
template <bool FUSED>
__device__ __forceinline__ uint64_t ra_flag_step(const RaArgs &a, uint32_t i, uint64_t *wave_tot)
{
  const uint32_t n = ra_n(a);
  unsigned long long pack = 0;
  if (i < n) {
    const uint32_t cell = a.arr_cell[i];
    const uint32_t r = cell != kRaNoCell ? a.rec[cell] : kRaNoRec;
    if (r != kRaNoRec) {
      const uint32_t fidx = a.arr_fidx[i];
      if (fidx < SG_MAX_BI_SIZE) {
        // rr_emplace_mbuf: the entry goes where its sequence number says
        a.tab[(size_t)r * SG_MAX_BI_SIZE + fidx] = (unsigned long long)a.arrivals[i] | ((unsigned long long)a.arr_len[i] << 32);
      } else {
        refuse(a.status, a.status_flag, kStBadTable);  // beyond what a request's tables hold (src/p2p_bufs.h:10)
      }
      const unsigned long long acc = ra_acc<FUSED>(a, cell);
      const uint32_t cnt = ra_cnt(acc);
      if (ra_word<FUSED>(a.last + cell) == i && ra_complete(a, cell, acc)) {
        if (cnt <= SG_MAX_BI_SIZE) pack = (1ull << 32) | cnt;
        else refuse(a.status, a.status_flag, kStBadTable);
      }
    }
  }
  uint64_t tot;
  const uint64_t ex = block_exclusive_scan<kRaBlock>(pack, wave_tot, &tot);
  if (i < n) a.arr_pack[i] = pack ? (ex | (1ull << 63)) : 0;  // top bit: "a request completes here"
  return tot;
}

__global__ __launch_bounds__(kRaBlock) void k_ra_flag(RaArgs a)
{
  __shared__ uint64_t wave_tot[kRaBlock / kWave];
  const uint64_t tot = ra_flag_step<false>(a, blockIdx.x * kRaBlock + threadIdx.x, wave_tot);
  if (threadIdx.x == 0) a.blk[blockIdx.x] = tot;
}

// One thread closes the call: counts, the free ring's head, the epoch.  `run` is the packed
// (requests, fragments) total of the call.  Returns whether the output tables overflowed.
template <bool FUSED>
__device__ __forceinline__ uint32_t ra_scan_finish(const RaArgs &a, uint64_t run)
{
  uint32_t n_req = (uint32_t)(run >> 32), n_frag = (uint32_t)run;
  uint32_t overflow = 0;
  if (n_req > a.max_req || n_frag > a.max_frag) {
    // the output tables cannot take what completed: nothing is emitted, the requests stay parked
    refuse(a.status, a.status_flag, kStBadTable);
    overflow = 1;
    n_req = n_frag = 0;
  }
  a.words[kRaOverflow] = overflow;
  // cells claimed since the last call: as far as the head has moved
  uint32_t head = ra_word<FUSED>(a.words + kRaHead);
  const uint32_t claims = head - a.words[kRaHeadSeen];
  // claims beyond the pool ran the head past the tail
  if ((int32_t)(head - a.words[kRaTail]) > 0) head = a.words[kRaTail];
  a.words[kRaHead] = head;
  a.words[kRaHeadSeen] = head;
  a.req_first[n_req] = n_frag;
  const uint32_t in_flight = a.words[kRaInFlight] + claims - n_req;
  const uint32_t dropped = ra_word<FUSED>(a.words + kRaDropped);
  a.words[kRaInFlight] = in_flight;
  a.words[kRaDropped] = 0;
  a.words[kRaEpoch] += 1;
  const uint32_t c[4] = {n_req, n_frag, dropped, in_flight};
  for (int k = 0; k < 4; k++) {
    if (a.counts_out) a.counts_out[k] = c[k];
    a.counts_host[k] = c[k];  // straight into pinned host memory: nothing to copy back
  }
  return overflow;
}

__global__ __launch_bounds__(kRaBlock) void k_ra_scan(RaArgs a)
{
  __shared__ uint64_t wave_tot[kRaBlock / kWave];
  const uint32_t n = ra_n(a);
  const uint32_t n_blocks = (n + kRaBlock - 1) / kRaBlock;
  uint64_t run = 0;
  for (uint32_t base = 0; base < n_blocks; base += kRaBlock) {
    const uint32_t b = base + threadIdx.x;
    const uint64_t v = b < n_blocks ? a.blk[b] : 0;
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan<kRaBlock>(v, wave_tot, &tot);
    if (b < n_blocks) a.blk[b] = run + ex;
    run += tot;
  }
  if (threadIdx.x == 0) (void)ra_scan_finish<false>(a, run);
}

// The wavefront of a completing arrival hands the request over: its record goes
// into the output tables in sequence order, the record is emptied and returned
// to the free ring, the cell is emptied.  The request's rank and first fragment
// index hang on that arrival (arr_pack there plus its workgroup's scanned total).
template <bool FUSED>
__device__ __forceinline__ void ra_emit_step(const RaArgs &a, uint32_t i, uint32_t *take, bool overflow)
{
  const uint32_t n = ra_n(a);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t cell = kRaNoCell;
  unsigned long long v = 0;
  bool completes = false;
  if (i < n) {
    cell = a.arr_cell[i];
    const unsigned long long p = a.arr_pack[i];
    completes = cell != kRaNoCell && (p >> 63) && !overflow;
    if (completes) v = (p & ~(1ull << 63)) + (FUSED ? 0ull : a.blk[i / kRaBlock]);  // one workgroup: nothing before it
    // the position of a request's last arrival counts per call
    if (cell != kRaNoCell && !completes) a.last[cell] = 0;
  }
  unsigned long long todo = __ballot(completes);
  // reap_rr for all of this workgroup's requests: one addition to the ring's tail
  const uint32_t tail0 = ra_block_take(&a.words[kRaTail], (uint32_t)__popcll(todo), take);
  // requests of a few fragments are handed over by the completing lane itself, all such lanes
  // at once; the wavefront then walks the larger ones together
  constexpr uint32_t kOwn = 8;
  const uint32_t my_rank = (uint32_t)__popcll(todo & ((1ull << lane) - 1ull));
  bool own = false;
  if (completes) {
    const uint32_t cnt = ra_cnt(ra_acc<FUSED>(a, cell));
    own = cnt <= kOwn;
    if (own) {
      const uint32_t r = (uint32_t)(v >> 32), first = (uint32_t)v, rc = a.rec[cell];
      unsigned long long *t = a.tab + (size_t)rc * SG_MAX_BI_SIZE;
      unsigned long long e[kOwn];
#pragma unroll
      for (uint32_t j = 0; j < kOwn; j++) e[j] = j < cnt ? t[j] : 0ull;
#pragma unroll
      for (uint32_t j = 0; j < kOwn; j++) {
        if (j < cnt) {
          a.frag_slot[first + j] = (uint32_t)e[j];
          a.frag_len[first + j] = (uint32_t)(e[j] >> 32);
          t[j] = 0;
        }
      }
      a.req_first[r] = first;
      if (a.req_token) a.req_token[r] = ra_key(a.keys + cell);
      if (a.req_hdr_slot) a.req_hdr_slot[r] = (uint32_t)e[0];
      a.free_ring[(tail0 + my_rank) & a.rmask] = rc;
      a.acc[cell] = 0;
      a.last[cell] = 0;
      a.want[cell] = 0;
      a.rec[cell] = kRaNoRec;
      __hip_atomic_store(&a.keys[cell], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  const unsigned long long all_done = todo;
  todo &= ~__ballot(own);
  while (todo) {
    const int l = __ffsll((long long)todo) - 1;
    todo &= todo - 1;
    const uint32_t nth = (uint32_t)__popcll(all_done & ((1ull << l) - 1ull));
    const uint32_t c = (uint32_t)__shfl((int)cell, l, kWave);
    const uint32_t r = (uint32_t)__shfl((int)(uint32_t)(v >> 32), l, kWave);
    const uint32_t first = (uint32_t)__shfl((int)(uint32_t)v, l, kWave);
    const uint32_t rc = a.rec[c], cnt = ra_cnt(ra_acc<FUSED>(a, c));
    unsigned long long *t = a.tab + (size_t)rc * SG_MAX_BI_SIZE;
    for (uint32_t j = lane; j < cnt; j += kWave) {
      const unsigned long long e = t[j];
      a.frag_slot[first + j] = (uint32_t)e;
      a.frag_len[first + j] = (uint32_t)(e >> 32);
      t[j] = 0;  // a fresh request finds an empty record
      if (j == 0) {
        a.req_first[r] = first;
        if (a.req_token) a.req_token[r] = ra_key(a.keys + c);
        if (a.req_hdr_slot) a.req_hdr_slot[r] = (uint32_t)e;  // the slot whose header the responses answer
      }
    }
    if (lane == 0) {
      // the record goes back to the free ring, the token leaves the table
      a.free_ring[(tail0 + nth) & a.rmask] = rc;
      a.acc[c] = 0;
      a.last[c] = 0;
      a.want[c] = 0;
      a.rec[c] = kRaNoRec;
      __hip_atomic_store(&a.keys[c], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

__global__ __launch_bounds__(kRaTakeBlock) void k_ra_emit(RaArgs a)
{
  __shared__ uint32_t take[kRaTakeBlock / kWave + 1];
  ra_emit_step<false>(a, blockIdx.x * kRaTakeBlock + threadIdx.x, take, a.words[kRaOverflow] != 0);
}

// A burst of at most kRaTakeBlock arrivals: the four steps by one workgroup in one launch.
static_assert(kRaTakeBlock == kRaBlock, "one workgroup size for all steps of a burst");
__global__ __launch_bounds__(kRaTakeBlock) void k_ra_burst(RaArgs a)
{
  __shared__ uint32_t take[kRaTakeBlock / kWave + 1];
  __shared__ uint64_t wave_tot[kRaBlock / kWave];
  __shared__ uint32_t overflow;
  const uint32_t i = threadIdx.x;
  ra_insert_step(a, i, take);
  __syncthreads();
  const uint64_t tot = ra_flag_step<true>(a, i, wave_tot);
  if (threadIdx.x == 0) overflow = ra_scan_finish<true>(a, tot);
  __syncthreads();
  ra_emit_step<true>(a, i, take, overflow != 0);
}

// Empties the table: every cell, every record, all records back in the ring.
__global__ __launch_bounds__(256) void k_ra_reset(RaArgs a, uint32_t cells, uint32_t records)
{
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < cells) {
    a.keys[i] = 0;
    a.acc[i] = 0;
    a.want[i] = a.last[i] = a.seen[i] = 0;
    a.rec[i] = kRaNoRec;
  }
  if (i < records) a.free_ring[i] = (uint32_t)i;
  if (i < (size_t)records * SG_MAX_BI_SIZE) a.tab[i] = 0;
  if (i < kRaWords) a.words[i] = i == kRaTail ? records : 0u;
}

// Drops the requests no fragment has come in for during the last max_age calls
// (a lost fragment parks its request for good in the reference,
// src/p2p_rpc_rr_pool_ng.h:57-64; here the caller can clear such requests out).
// One wavefront per cell.
__global__ __launch_bounds__(256) void k_ra_evict(RaArgs a, uint32_t cells, uint32_t max_age)
{
  const uint32_t c = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  if (c >= cells) return;
  if (a.keys[c] == 0ull) return;
  if (a.words[kRaEpoch] - a.seen[c] <= max_age) return;
  const uint32_t rc = a.rec[c];
  if (rc != kRaNoRec) {
    unsigned long long *t = a.tab + (size_t)rc * SG_MAX_BI_SIZE;
    for (uint32_t j = lane; j < SG_MAX_BI_SIZE; j += kWave) t[j] = 0;
  }
  if (lane == 0) {
    if (rc != kRaNoRec) {
      const uint32_t tl = atomicAdd(&a.words[kRaTail], 1u);
      a.free_ring[tl & a.rmask] = rc;
    }
    a.acc[c] = 0;
    a.last[c] = 0;
    a.want[c] = 0;
    a.rec[c] = kRaNoRec;
    a.keys[c] = 0;
    atomicSub(&a.words[kRaInFlight], 1u);
    atomicAdd(&a.words[kRaEvicted], 1u);
  }
}

// Sets `n` 32-bit words to zero (a fill kernel rather than a memset node, so
// that callers may record the launch into a graph).
__global__ __launch_bounds__(kBlock) void k_zero_words(uint32_t *p, uint32_t n)
{
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace

// ---------------------------------------------------------------------------
// scratch of the allocation-free entry point
// ---------------------------------------------------------------------------
// One array per GPU the library runs on, held until the process ends.  Host
// code never uses the array's name as an address: the address on each device
// comes from hipGetSymbolAddress (static_scratch_of below).
namespace {
constexpr size_t kStaticDesc = sizeof(u32x4) * (size_t)SG_STATIC_MAX_FRAMES;
constexpr size_t kStaticReq = sizeof(uint64_t) * (size_t)SG_STATIC_MAX_REQS;
constexpr size_t kStaticTile = sizeof(uint64_t) * (SG_STATIC_MAX_REQS / kPartMin + 2);
constexpr size_t kStaticWords = 256;  // cursors, staged cursors, status, refusal flag
constexpr size_t kStaticBytes = kStaticDesc + 2 * kStaticReq + kStaticTile + kStaticWords;
}  // namespace
static __device__ __align__(256) uint8_t scratch[kStaticBytes];

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct EvPair {
  hipEvent_t a, b;
  int which;
};

// Device memory a batched call works in, beyond its inputs and outputs.  A
// context owns one set (allocated at creation); the allocation-free entry
// point uses a set carved out of a static device array.
struct Scratch {
  uint32_t max_reqs = 0, max_frames = 0;
  u32x4 *desc = nullptr;         // run descriptors, max_frames
  uint64_t *req_size = nullptr;  // max_reqs
  uint64_t *req_off = nullptr;   // max_reqs
  uint64_t *tile_tot = nullptr;  // one total per kScanTile requests, for the tiled request scan
  // bump-ring cursors (request arena, response arena) and the values a
  // descriptor pass stages for the copy kernel to commit
  uint64_t *cursor[2] = {nullptr, nullptr};
  uint64_t *next_cursor[2] = {nullptr, nullptr};
  uint32_t *slot_idx[2] = {nullptr, nullptr};  // next slot of the application ring to fill / to serve
  uint32_t *desc_tag = nullptr;    // {generation, requests, items} of the descriptors in `desc`
  uint32_t *desc_gen = nullptr;    // host counter behind the generation (one per scratch)
  uint32_t *csum_part = nullptr;   // kPartStride words per frame (two-phase UDP checksum of long frames)
  uint32_t *csum_valid = nullptr;  // one mark per frame, zero between calls
  uint32_t *status = nullptr;
  volatile uint32_t *flag = nullptr;  // raised with every refusal (pinned host memory in a context)
};

struct sg_hip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool own_stream = false;
  uint32_t max_reqs = 0, max_frames = 0;
  // device scratch
  u32x4 *desc = nullptr;
  uint64_t *req_size = nullptr;
  uint64_t *req_off = nullptr;
  uint64_t *tile_tot = nullptr;  // one total per 4096 requests, for the tiled request scan
  // [0] request-arena cursor, [1] response-arena cursor, [2], [3] their staged successors
  uint64_t *cursors = nullptr;
  uint32_t *csum_scratch = nullptr;  // csum_part and csum_valid
  uint32_t desc_gen = 0;
  uint32_t *status = nullptr;
  Scratch sc;
  // pinned staging for the per-request entry points (device reads it in place)
  Run *h_runs = nullptr;
  uint32_t h_runs_cap = 0;
  uint64_t *h_ptrs = nullptr;
  uint32_t *h_status = nullptr;  // pinned: [0] copy of status (read back only after a refusal), [1] the refusal flag
  volatile uint32_t *h_flag = nullptr;
  // profiling
  bool profiling = false;
  std::vector<EvPair> ev_used, ev_free;
  double prof_ms[6] = {0, 0, 0, 0, 0, 0};
  uint64_t prof_n[6] = {0, 0, 0, 0, 0, 0};
  // reassembly scratch, allocated by the first sg_hip_reassemble call
  void *ra_mem = nullptr;
  uint32_t ra_cells = 0;    // cells of the request table (power of two >= 4 * max_reqs)
  uint32_t ra_records = 0;  // records of the pool (power of two >= max_reqs)
  uint32_t *h_counts = nullptr;  // pinned: requests, fragments, dropped, in flight (written by k_ra_scan itself)
  char err[512] = {0};
};

static char g_create_err[512];

static int fail(sg_hip_ctx *c, int code, const char *fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(c ? c->err : g_create_err, 512, fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(c, call)                                                                      \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess)                                                                     \
      return fail((c), SG_E_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),       \
                  __FILE__, __LINE__);                                                        \
  } while (0)

namespace {

struct DeviceGuard {
  int prev = -1;
  bool ok = false;
  explicit DeviceGuard(int dev)
  {
    if (hipGetDevice(&prev) == hipSuccess) {
      if (prev == dev) ok = true;
      else ok = hipSetDevice(dev) == hipSuccess;
    }
  }
  ~DeviceGuard()
  {
    if (ok && prev >= 0) (void)hipSetDevice(prev);
  }
};

uint32_t hdr_len_of(uint32_t profile) { return profile == SG_HDR_REF64 ? 64u : 58u; }

int check_ring(sg_hip_ctx *c, const sg_ring_desc &r, const char *what)
{
  if (!r.base || r.n_slots == 0) return fail(c, SG_E_INVAL, "%s ring: null base or no slots", what);
  if (r.hdr_profile > SG_HDR_REF64) return fail(c, SG_E_INVAL, "%s ring: unknown header profile %u", what, r.hdr_profile);
  if (r.slot_size < hdr_len_of(r.hdr_profile) || (r.slot_size & 1u))
    return fail(c, SG_E_INVAL, "%s ring: slot size %u must be even and hold a header", what, r.slot_size);
  if ((uintptr_t)r.base & 1u) return fail(c, SG_E_INVAL, "%s ring: base address must be even", what);
  return SG_OK;
}

int check_app(sg_hip_ctx *c, const sg_app_desc &a, AppDev *out, uint64_t *max_req_bytes)
{
  if (a.n_tensors > SG_MAX_TENSORS) return fail(c, SG_E_INVAL, "n_tensors %u > %d", a.n_tensors, SG_MAX_TENSORS);
  memset(out, 0, sizeof *out);
  out->n_tensors = a.n_tensors;
  *max_req_bytes = 0;
  if (a.n_tensors == 0) {
    if (!a.arena || a.arena_cap == 0) return fail(c, SG_E_INVAL, "packed mode needs an arena and a capacity");
    out->arena = static_cast<uint8_t *>(a.arena);
    out->cap = a.arena_cap;
    out->mirrored = a.arena_mirrored ? 1u : 0u;
    return SG_OK;
  }
  for (uint32_t t = 0; t < a.n_tensors; t++) {
    if (!a.tensor_base[t] || a.tensor_size[t] == 0)
      return fail(c, SG_E_INVAL, "tensor %u: null base or zero size", t);
    out->tensor_base[t] = static_cast<uint8_t *>(a.tensor_base[t]);
    out->tensor_size[t] = a.tensor_size[t];
    *max_req_bytes += a.tensor_size[t];
  }
  return SG_OK;
}

// Launch geometry for one wavefront per item; with the XCD-aware order the
// grid is padded to whole rounds of kXcds * kXcdRun workgroups.
void geometry(uint64_t n_waves, bool want_remap, uint32_t *grid, uint32_t *remap)
{
  const uint32_t groups = (uint32_t)((n_waves + kWavesPerBlock - 1) / kWavesPerBlock);
  const uint32_t round = kXcds * kXcdRun;
  if (want_remap && groups >= 2 * round) {
    *grid = (groups + round - 1) / round * round;
    *remap = 1;
  } else {
    *grid = groups;
    *remap = 0;
  }
}

int prof_begin(sg_hip_ctx *c, int which)
{
  if (!c || !c->profiling) return SG_OK;
  EvPair p;
  if (!c->ev_free.empty()) {
    p = c->ev_free.back();
    c->ev_free.pop_back();
  } else {
    HIP_TRY(c, hipEventCreate(&p.a));
    HIP_TRY(c, hipEventCreate(&p.b));
  }
  p.which = which;
  HIP_TRY(c, hipEventRecord(p.a, c->stream));
  c->ev_used.push_back(p);
  return SG_OK;
}

int prof_end(sg_hip_ctx *c)
{
  if (!c || !c->profiling) return SG_OK;
  HIP_TRY(c, hipEventRecord(c->ev_used.back().b, c->stream));
  return SG_OK;
}

int prof_drain(sg_hip_ctx *c)
{
  for (EvPair &p : c->ev_used) {
    float ms = 0.f;
    HIP_TRY(c, hipEventElapsedTime(&ms, p.a, p.b));
    c->prof_ms[p.which] += ms;
    c->prof_n[p.which] += 1;
    c->ev_free.push_back(p);
  }
  c->ev_used.clear();
  return SG_OK;
}

// Descriptor build: kernel shape by the average request, then the bump-ring
// scan of the request totals where offsets are not plain multiples.
int launch_prep(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const PrepArgs &args)
{
  int rc = prof_begin(c, 0);
  if (rc != SG_OK) return rc;
  PrepArgs p = args;
  const uint32_t avg = p.n_items / p.n_req;
  const bool tiled = p.packed && !p.fixed_offsets && !(p.n_req <= 2 * kScanTile || p.counts);
  // requests per entry of the workgroup sums k_prep_group leaves for the tiled scan
  const uint32_t per_part = avg <= 8 ? 4 * kWavesPerBlock : avg <= 16 ? 2 * kWavesPerBlock : 0;
  if (tiled && per_part) p.part = sc.tile_tot;
  if (avg <= 8) {
    k_prep_group<16><<<(p.n_req + 4 * kWavesPerBlock - 1) / (4 * kWavesPerBlock), kBlock, 0, st>>>(p);
  } else if (avg <= 16) {
    k_prep_group<32><<<(p.n_req + 2 * kWavesPerBlock - 1) / (2 * kWavesPerBlock), kBlock, 0, st>>>(p);
  } else if (avg <= 32) {
    k_prep_wave<<<(p.n_req + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, st>>>(p);
  } else if (avg <= 256) {
    k_prep_block<256><<<p.n_req, 256, 0, st>>>(p);
  } else {
    k_prep_block<1024><<<p.n_req, 1024, 0, st>>>(p);
  }
  if (p.packed && !p.fixed_offsets) {
    if (p.n_req <= 2 * kScanTile || p.counts) {  // counts on the device: one workgroup walks whatever is there
      k_req_scan<<<1, kScanBlock, 0, st>>>(p);
    } else {
      const uint32_t n_tiles = (p.n_req + kScanTile - 1) / kScanTile;
      if (p.part) {
        k_req_scan_parts<<<n_tiles, kScanBlock, 0, st>>>(p, per_part, n_tiles);
      } else {
        // (one launch in which every workgroup adds up the REQUEST sizes before its tile by itself
        // was measured at 32768 requests: 30.6 us for the descriptor pass against 26.9 us with these)
        k_req_scan_local<<<n_tiles, kScanBlock, 0, st>>>(p, sc.tile_tot);
        k_req_scan_add<<<n_tiles, kScanBlock, 0, st>>>(p, sc.tile_tot, n_tiles);
      }
    }
  }
  return prof_end(c);
}

// Behind the copy kernel: advance the cursor (single-kernel calls on a packed
// arena) and publish slot states (where the caller keeps a slot ring).
void launch_finish(const Scratch &sc, hipStream_t st, uint64_t *cursor, uint64_t size, uint64_t cap, uint32_t n_req,
                   const uint32_t *counts, uint32_t *state, uint32_t n_states, int which, bool all_or_nothing)
{
  if (!cursor && !state) return;
  FinishArgs f;
  memset(&f, 0, sizeof f);
  f.cursor = cursor;
  f.size = size;
  f.cap = cap;
  f.n_req = n_req;
  f.counts = counts;
  f.state = state;
  f.n_states = n_states;
  f.slot_idx = sc.slot_idx[which];
  // gather fills FREE slots and publishes RX_COMPLETE; scatter serves WORK_COMPLETE slots and
  // frees them (src/splitrpc_server/p2p_rpc_dpdk_server.cc:130,175; states src/p2p_rpc_app_ctx.h:22)
  f.expect = which == 0 ? SG_SLOT_FREE : SG_SLOT_WORK_COMPLETE;
  f.publish = which == 0 ? SG_SLOT_RX_COMPLETE : SG_SLOT_FREE;
  f.all_or_nothing = all_or_nothing ? 1u : 0u;
  f.status = sc.status;
  f.status_flag = sc.flag;
  k_finish<<<1, kBlock, 0, st>>>(f);
}

int finish(sg_hip_ctx *c, uint32_t flags)
{
  HIP_TRY(c, hipGetLastError());
  if (!c) return SG_OK;  // allocation-free entry point: launches only
  if (flags & SG_F_ASYNC) {
    // keep the event list bounded on long asynchronous runs
    if (c->profiling && c->ev_used.size() > 4096) return sg_hip_sync(c);
    return SG_OK;
  }
  return sg_hip_sync(c);
}

}  // namespace

// floor(n / d) == (n * M) >> (27 + l) for every n < 2^27, with l = ceil(log2 d), M = ceil(2^(27 + l) / d)
// Walks the tensor-major buffers once per fragment index (all requests of the call have `size`
// bytes cut at `mtu`): where fragment i lands, for every i.  Returns the number of entries, or 0
// when there is no plan (more fragments per request than entries, a tensor of 4 GiB or more per
// request).
static uint32_t fill_plan(const AppDev &app, uint64_t size, uint32_t mtu, uint64_t per, FragPlan *plan)
{
  if (per > kPlanMax) return 0;
  for (uint32_t t = 0; t < app.n_tensors; t++)
    if (app.tensor_size[t] > 0xffffffffull) return 0;
  for (uint32_t i = 0; i < per; i++) {
    const uint64_t off = (uint64_t)i * mtu;
    const uint64_t len = size - off < mtu ? size - off : mtu;
    FragPlan &fp = plan[i];
    memset(&fp, 0, sizeof fp);
    fp.kind = 2;
    uint64_t t0 = 0;
    for (uint32_t t = 0; t < app.n_tensors; t++) {
      const uint64_t t1 = t0 + app.tensor_size[t];
      if (off < t1) {
        fp.base_a = (uint64_t)(uintptr_t)app.tensor_base[t] + (off - t0);
        fp.stride_a = (uint32_t)app.tensor_size[t];
        if (off + len <= t1) {
          fp.kind = 0;
          fp.len_a = (uint32_t)len;
        } else if (t + 1 < app.n_tensors && off + len <= t1 + app.tensor_size[t + 1]) {
          fp.kind = 1;
          fp.len_a = (uint32_t)(t1 - off);
          fp.base_b = (uint64_t)(uintptr_t)app.tensor_base[t + 1];
          fp.stride_b = (uint32_t)app.tensor_size[t + 1];
        }
        break;
      }
      t0 = t1;
    }
  }
  return (uint32_t)per;
}

static void magic_div(uint64_t d, uint32_t *mul, uint32_t *shift)
{
  uint32_t l = 0;
  while ((1ull << l) < d) l++;
  *shift = 27 + l;
  *mul = (uint32_t)(((1ull << *shift) + d - 1) / d);
}

// Lanes a short frame of at most `bytes` payload bytes is given (two steps of L - 1
// chunks without looping), or 0 where a whole wavefront per frame is the better deal.
static uint32_t small_lanes(uint64_t bytes)
{
  if (bytes <= 2 * 15 * 16) return 16;
  if (bytes <= 2 * 31 * 16) return 32;
  return 0;
}

// Remainder fragments get wavefronts of their own kind when they are a good share of the
// call's wavefronts -- and, where that takes a launch of its own (scatter), when the call is
// large enough to hide one more launch.
static bool small_last_pays(uint64_t per_req, uint32_t n_req, uint32_t flags, bool own_launch)
{
  if (per_req < 2) return false;
  return (flags & SG_F_FORCE_SMALL) || (per_req <= 8 && (!own_launch || n_req >= 1024));
}

static void launch_scatter_small(hipStream_t st, const ScatterArgs &sa, uint32_t lanes, uint32_t n_frames, bool full_csum)
{
  const uint32_t per_wave = kWave / lanes;
  const uint32_t grid = (n_frames + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
  if (lanes == 16 && full_csum) k_scatter_small<16, true><<<grid, kBlock, 0, st>>>(sa);
  else if (lanes == 16) k_scatter_small<16, false><<<grid, kBlock, 0, st>>>(sa);
  else if (full_csum) k_scatter_small<32, true><<<grid, kBlock, 0, st>>>(sa);
  else k_scatter_small<32, false><<<grid, kBlock, 0, st>>>(sa);
}

// Long frames with the full UDP checksum go to several wavefronts per frame when the
// scratch has room for their sums (k_scatter<.., DEFER> + k_udp_finish).
static bool csum_in_two_phases(const Scratch &sc, uint32_t pieces, bool full_csum)
{
  return full_csum && pieces > 1 && pieces + 1 <= kPartStride && sc.csum_part != nullptr;
}

template <bool FUSED>
static void launch_scatter(hipStream_t st, const ScatterArgs &sa, uint32_t grid, bool full_csum, bool defer = false)
{
  const bool lng = sa.pieces > 1;
  if (defer) {
    k_scatter<true, FUSED, true, true><<<grid, kBlock, 0, st>>>(sa);
    k_udp_finish<FUSED><<<(sa.n_items + kBlock - 1) / kBlock, kBlock, 0, st>>>(sa);
  } else if (full_csum && lng) k_scatter<true, FUSED, true><<<grid, kBlock, 0, st>>>(sa);
  else if (full_csum) k_scatter<true, FUSED, false><<<grid, kBlock, 0, st>>>(sa);
  else if (lng) k_scatter<false, FUSED, true><<<grid, kBlock, 0, st>>>(sa);
  else k_scatter<false, FUSED, false><<<grid, kBlock, 0, st>>>(sa);
}

extern "C" {

int sg_hip_abi_version(void) { return SG_HIP_ABI_VERSION; }

const char *sg_hip_last_error(const sg_hip_ctx *ctx) { return ctx ? ctx->err : g_create_err; }

void *sg_hip_stream(sg_hip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

static int create_impl(sg_hip_ctx *c, int device_id, const sg_hip_cfg *cfg)
{
  int n_dev = 0;
  HIP_TRY(nullptr, hipGetDeviceCount(&n_dev));
  if (device_id < 0 || device_id >= n_dev)
    return fail(nullptr, SG_E_INVAL, "device %d not present (%d devices)", device_id, n_dev);
  c->device = device_id;
  DeviceGuard g(device_id);
  if (!g.ok) return fail(nullptr, SG_E_HIP, "cannot select device %d", device_id);
  hipDeviceProp_t prop;
  HIP_TRY(nullptr, hipGetDeviceProperties(&prop, device_id));
  if (prop.warpSize != (int)kWave)
    return fail(nullptr, SG_E_INVAL, "device %d has %d-wide wavefronts; this library is built for 64", device_id, prop.warpSize);
  c->max_reqs = cfg && cfg->max_reqs ? cfg->max_reqs : 4096u;
  c->max_frames = cfg && cfg->max_frames ? cfg->max_frames : 65536u;
  if (cfg && cfg->stream) {
    c->stream = static_cast<hipStream_t>(cfg->stream);
  } else {
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    c->own_stream = true;
  }
  HIP_TRY(nullptr, hipMalloc(&c->desc, sizeof(u32x4) * (size_t)c->max_frames));
  HIP_TRY(nullptr, hipMalloc(&c->req_size, sizeof(uint64_t) * (size_t)c->max_reqs));
  HIP_TRY(nullptr, hipMalloc(&c->req_off, sizeof(uint64_t) * (size_t)c->max_reqs));
  HIP_TRY(nullptr, hipMalloc(&c->tile_tot, sizeof(uint64_t) * ((size_t)c->max_reqs / kPartMin + 2)));
  HIP_TRY(nullptr, hipMalloc(&c->cursors, 7 * sizeof(uint64_t)));  // [4]: the two slot indices, [5], [6]: descriptor tag
  HIP_TRY(nullptr, hipMalloc(&c->status, sizeof(uint32_t)));
  HIP_TRY(nullptr, hipMalloc(&c->csum_scratch, sizeof(uint32_t) * (size_t)c->max_frames * (kPartStride + 1)));
  HIP_TRY(nullptr, hipMemsetAsync(c->csum_scratch, 0, sizeof(uint32_t) * (size_t)c->max_frames * (kPartStride + 1), c->stream));
  HIP_TRY(nullptr, hipMemsetAsync(c->cursors, 0, 7 * sizeof(uint64_t), c->stream));
  HIP_TRY(nullptr, hipMemsetAsync(c->status, 0, sizeof(uint32_t), c->stream));
  c->h_runs_cap = 8192;
  HIP_TRY(nullptr, hipHostMalloc(&c->h_runs, sizeof(Run) * c->h_runs_cap, hipHostMallocDefault));
  HIP_TRY(nullptr, hipHostMalloc(&c->h_ptrs, sizeof(uint64_t) * (SG_MAX_BI_SIZE + 8), hipHostMallocDefault));
  HIP_TRY(nullptr, hipHostMalloc(&c->h_status, 2 * sizeof(uint32_t), hipHostMallocDefault));
  c->h_status[0] = c->h_status[1] = 0;
  c->h_flag = c->h_status + 1;
  HIP_TRY(nullptr, hipStreamSynchronize(c->stream));
  Scratch &sc = c->sc;
  sc.max_reqs = c->max_reqs;
  sc.max_frames = c->max_frames;
  sc.desc = c->desc;
  sc.req_size = c->req_size;
  sc.req_off = c->req_off;
  sc.tile_tot = c->tile_tot;
  sc.cursor[0] = c->cursors + 0;
  sc.cursor[1] = c->cursors + 1;
  sc.next_cursor[0] = c->cursors + 2;
  sc.next_cursor[1] = c->cursors + 3;
  sc.slot_idx[0] = reinterpret_cast<uint32_t *>(c->cursors + 4);
  sc.slot_idx[1] = sc.slot_idx[0] + 1;
  sc.desc_tag = reinterpret_cast<uint32_t *>(c->cursors + 5);
  sc.desc_gen = &c->desc_gen;
  sc.csum_part = c->csum_scratch;
  sc.csum_valid = c->csum_scratch + (size_t)c->max_frames * kPartStride;
  sc.status = c->status;
  sc.flag = c->h_flag;
  return SG_OK;
}

sg_hip_ctx *sg_hip_create(int device_id, const sg_hip_cfg *cfg)
{
  g_create_err[0] = 0;
  if (cfg && cfg->struct_size != sizeof(sg_hip_cfg)) {
    fail(nullptr, SG_E_INVAL, "sg_hip_cfg.struct_size %u != %zu", cfg->struct_size, sizeof(sg_hip_cfg));
    return nullptr;
  }
  sg_hip_ctx *c = new (std::nothrow) sg_hip_ctx();
  if (!c) {
    fail(nullptr, SG_E_NOMEM, "out of host memory");
    return nullptr;
  }
  if (create_impl(c, device_id, cfg) != SG_OK) {
    sg_hip_destroy(c);
    return nullptr;
  }
  return c;
}

void sg_hip_destroy(sg_hip_ctx *c)
{
  if (!c) return;
  DeviceGuard g(c->device);
  if (c->stream) (void)hipStreamSynchronize(c->stream);
  for (EvPair &p : c->ev_used) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  for (EvPair &p : c->ev_free) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  (void)hipFree(c->desc);
  (void)hipFree(c->req_size);
  (void)hipFree(c->req_off);
  (void)hipFree(c->tile_tot);
  (void)hipFree(c->cursors);
  (void)hipFree(c->csum_scratch);
  (void)hipFree(c->status);
  if (c->h_runs) (void)hipHostFree(c->h_runs);
  if (c->h_ptrs) (void)hipHostFree(c->h_ptrs);
  if (c->h_status) (void)hipHostFree(c->h_status);
  if (c->h_counts) (void)hipHostFree(c->h_counts);
  (void)hipFree(c->ra_mem);
  if (c->own_stream && c->stream) (void)hipStreamDestroy(c->stream);
  delete c;
}

int sg_hip_sync(sg_hip_ctx *c)
{
  if (!c) return SG_E_INVAL;
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  int rc = prof_drain(c);
  if (rc != SG_OK) return rc;
  if (*c->h_flag) {
    // the rare path: fetch the bits, then clear both words
    HIP_TRY(c, hipMemcpyAsync(c->h_status, c->status, sizeof(uint32_t), hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, hipMemsetAsync(c->status, 0, sizeof(uint32_t), c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    *c->h_flag = 0;
    const uint32_t st = c->h_status[0];
    return fail(c, SG_E_DATA, "kernel refused input:%s%s%s%s%s%s%s%s",
                (st & kStBadSlot) ? " slot index beyond ring;" : "",
                (st & kStBadLen) ? " fragment longer than a slot holds;" : "",
                (st & kStBadSize) ? " request larger than its destination;" : "",
                (st & kStBadFrames) ? " frame count disagrees with size/mtu;" : "",
                (st & kStBadTable) ? " CSR table does not tile the items;" : "",
                (st & kStNotRule) ? " a fragment's length departs from the fragmenting rule;" : "",
                (st & kStSlotState) ? " an application slot was not in the state the call expects;" : "",
                (st & kStPoolFull) ? " more requests in flight than the reassembly pool holds;" : "");
  }
  return SG_OK;
}

int sg_hip_set_cursor(sg_hip_ctx *c, int which, uint64_t value)
{
  if (!c || which < 0 || which > 1) return fail(c, SG_E_INVAL, "cursor index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(c->cursors + which, &value, sizeof value, hipMemcpyHostToDevice));
  return SG_OK;
}

int sg_hip_get_cursor(sg_hip_ctx *c, int which, uint64_t *value)
{
  if (!c || !value || which < 0 || which > 1) return fail(c, SG_E_INVAL, "cursor index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(value, c->cursors + which, sizeof *value, hipMemcpyDeviceToHost));
  return SG_OK;
}

int sg_hip_set_slot_index(sg_hip_ctx *c, int which, uint32_t value)
{
  if (!c || which < 0 || which > 1) return fail(c, SG_E_INVAL, "slot index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(c->sc.slot_idx[which], &value, sizeof value, hipMemcpyHostToDevice));
  return SG_OK;
}

int sg_hip_get_slot_index(sg_hip_ctx *c, int which, uint32_t *value)
{
  if (!c || !value || which < 0 || which > 1) return fail(c, SG_E_INVAL, "slot index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(value, c->sc.slot_idx[which], sizeof *value, hipMemcpyDeviceToHost));
  return SG_OK;
}

int sg_hip_set_profiling(sg_hip_ctx *c, int on)
{
  if (!c) return SG_E_INVAL;
  int rc = sg_hip_sync(c);
  c->profiling = on != 0;
  for (int i = 0; i < 6; i++) { c->prof_ms[i] = 0; c->prof_n[i] = 0; }
  return rc;
}

int sg_hip_kernel_time(sg_hip_ctx *c, int which, double *total_ms, uint64_t *launches)
{
  if (!c || which < 0 || which > 5) return fail(c, SG_E_INVAL, "kernel index %d", which);
  int rc = sg_hip_sync(c);
  if (total_ms) *total_ms = c->prof_ms[which];
  if (launches) *launches = c->prof_n[which];
  return rc;
}

// ---- per-request ------------------------------------------------------------

// Runs longer than this are cut so that no single wavefront walks megabytes.
static const uint64_t kRunChunk = 16384;

static int copy_skb(sg_hip_ctx *c, const sg_sk_buf *skb)
{
  if (!c || !skb) return fail(c, SG_E_INVAL, "null argument");
  if (skb->num_items > SG_MAX_BI_SIZE - 1)
    return fail(c, SG_E_INVAL, "run table holds %llu runs; len[] has room for %d",
                (unsigned long long)skb->num_items, SG_MAX_BI_SIZE - 1);
  DeviceGuard g(c->device);
  // the pinned staging buffer is reused: the previous launch must have read it
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  uint32_t n = 0;
  for (uint64_t i = 0; i < skb->num_items; i++) {
    uint64_t src = skb->i_buf[i], dst = skb->o_buf[i], len = skb->len[i];
    if (len && (!src || !dst)) return fail(c, SG_E_INVAL, "run %llu has a null address", (unsigned long long)i);
    while (len) {
      uint64_t piece = len;
      if (piece > kRunChunk) {
        // cut where the destination is 16-byte aligned so later pieces need no head bytes
        piece = kRunChunk - (dst & 15u);
      }
      if (n == c->h_runs_cap) {
        // flush what is staged and start over
        int rc = prof_begin(c, 3);
        if (rc != SG_OK) return rc;
        k_copy_runs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(c->h_runs, n);
        rc = prof_end(c);
        if (rc != SG_OK) return rc;
        HIP_TRY(c, hipStreamSynchronize(c->stream));
        n = 0;
      }
      c->h_runs[n++] = Run{src, dst, piece};
      src += piece; dst += piece; len -= piece;
    }
  }
  if (n) {
    int rc = prof_begin(c, 3);
    if (rc != SG_OK) return rc;
    k_copy_runs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(c->h_runs, n);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  return finish(c, 0);
}

int sg_hip_gather(sg_hip_ctx *c, const sg_sk_buf *skb) { return copy_skb(c, skb); }
int sg_hip_scatter(sg_hip_ctx *c, const sg_sk_buf *skb) { return copy_skb(c, skb); }

static int fill_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, const uint8_t *tmpl, uint64_t token,
                     uint32_t profile, uint64_t payload_size, uint32_t mtu, uint32_t flags)
{
  if (!c || !hdrs) return fail(c, SG_E_INVAL, "null argument");
  if (profile > SG_HDR_REF64) return fail(c, SG_E_INVAL, "unknown header profile %u", profile);
  if (hdrs->num_items > SG_MAX_BI_SIZE) return fail(c, SG_E_INVAL, "header table holds %u entries", hdrs->num_items);
  if (mtu == 0) return fail(c, SG_E_INVAL, "mtu is zero");
  if (flags & SG_F_UDP_CSUM_FULL) return fail(c, SG_E_INVAL, "a header-only rewrite cannot finish the UDP checksum");
  const uint32_t n = hdrs->num_items;
  if (n == 0) return SG_OK;
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  for (uint32_t i = 0; i < n; i++) {
    if (!hdrs->burst_items[i]) return fail(c, SG_E_INVAL, "header %u is null", i);
    c->h_ptrs[i] = hdrs->burst_items[i];
  }
  // the template rides behind the pointer table in the same pinned block
  const uint8_t *d_tmpl = nullptr;
  if (tmpl) {
    memcpy(c->h_ptrs + SG_MAX_BI_SIZE, tmpl, 64);
    d_tmpl = reinterpret_cast<const uint8_t *>(c->h_ptrs + SG_MAX_BI_SIZE);
  }
  int rc = prof_begin(c, 4);
  if (rc != SG_OK) return rc;
  k_swap_hdrs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(
      c->h_ptrs, n, hdr_len_of(profile), profile == SG_HDR_REF64, flags & 0xfu, payload_size, mtu,
      d_tmpl, token);
  rc = prof_end(c);
  if (rc != SG_OK) return rc;
  return finish(c, 0);
}

int sg_hip_swap_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, uint32_t profile, uint64_t payload_size,
                     uint32_t mtu, uint32_t flags)
{
  return fill_hdrs(c, hdrs, nullptr, 0, profile, payload_size, mtu, flags);
}

int sg_hip_set_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, const uint8_t *hdr_template, uint64_t req_token,
                    uint32_t profile, uint64_t payload_size, uint32_t mtu, uint32_t flags)
{
  if (!hdr_template) return fail(c, SG_E_INVAL, "null header template");
  return fill_hdrs(c, hdrs, hdr_template, req_token, profile, payload_size, mtu, flags);
}

// ---- batched ------------------------------------------------------------------

// The gather call proper.  `c` may be null (allocation-free entry point): then
// errors go to the creation-error text, nothing is profiled and nothing waits.
static int gather_impl(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const sg_gather_args *a)
{
  int rc = check_ring(c, a->ring, "rx");
  if (rc != SG_OK) return rc;
  if (a->n_req == 0) return SG_OK;
  if (a->n_req > sc.max_reqs) return fail(c, SG_E_INVAL, "n_req %u > max_reqs %u", a->n_req, sc.max_reqs);
  if (a->n_frags > sc.max_frames) return fail(c, SG_E_INVAL, "n_frags %u > max_frames %u", a->n_frags, sc.max_frames);
  if ((!a->frag_slot && a->n_frags) || !a->req_first) return fail(c, SG_E_INVAL, "null fragment tables");
  if (!a->frag_len && a->n_frags && a->ring.hdr_profile != SG_HDR_BL58)
    return fail(c, SG_E_INVAL, "REF64 headers carry no payload length: frag_len is required");
  AppDev app;
  uint64_t max_req_bytes;
  rc = check_app(c, a->app, &app, &max_req_bytes);
  if (rc != SG_OK) return rc;
  const bool packed = app.n_tensors == 0;
  if (a->slot_state && a->n_slot_states == 0) return fail(c, SG_E_INVAL, "a slot ring of no slots");
  if (a->slot_state && a->n_req > a->n_slot_states)
    return fail(c, SG_E_INVAL, "%u requests do not fit a ring of %u application slots", a->n_req, a->n_slot_states);
  // a batch larger than the arena would lap itself and its wavefronts would race for the same bytes
  if (packed && a->fixed_req_size && (uint64_t)a->n_req * a->fixed_req_size > app.cap)
    return fail(c, SG_E_INVAL, "%u requests of %llu bytes do not fit an arena of %llu bytes", a->n_req,
                (unsigned long long)a->fixed_req_size, (unsigned long long)app.cap);

  const uint32_t hl0 = hdr_len_of(a->ring.hdr_profile);
  if (a->flags & SG_F_RULE_FRAGS) {
    // one size, cut by the rule: no descriptor pass, the copy kernel derives everything
    if (!a->fixed_req_size || !a->mtu) return fail(c, SG_E_INVAL, "SG_F_RULE_FRAGS needs fixed_req_size and mtu");
    if ((uint64_t)a->mtu + hl0 > a->ring.slot_size) return fail(c, SG_E_INVAL, "mtu %u + %u header bytes does not fit a %u-byte slot", a->mtu, hl0, a->ring.slot_size);
    const uint64_t per = (a->fixed_req_size + a->mtu - 1) / a->mtu;
    // with the counts on the device n_req and n_frags are bounds: the launch covers per * n_req fragments
    if (a->counts ? per * a->n_req > sc.max_frames : per * a->n_req != a->n_frags)
      return fail(c, SG_E_INVAL, "%u requests of %llu bytes at mtu %u are %llu fragments, not %u", a->n_req, (unsigned long long)a->fixed_req_size, a->mtu, (unsigned long long)(per * a->n_req), a->n_frags);
    const uint32_t n_items = (uint32_t)(per * a->n_req);
    if (n_items >= (1u << 27)) return fail(c, SG_E_INVAL, "%u fragments in one call: the limit is 2^27 - 1", n_items);
    if (a->fixed_req_size > 0xffffffffull || (packed ? a->fixed_req_size > app.cap : a->fixed_req_size > max_req_bytes))
      return fail(c, SG_E_INVAL, "request size %llu does not fit its destination", (unsigned long long)a->fixed_req_size);
    GatherRuleArgs ga;
    memset(&ga, 0, sizeof ga);
    ga.ring = static_cast<const uint8_t *>(a->ring.base);
    ga.frag_slot = a->frag_slot;
    ga.dst = packed ? app.arena : app.tensor_base[0];
    ga.cursor = sc.cursor[0];
    ga.size = a->fixed_req_size;
    ga.cap = packed ? app.cap : 0;
    ga.n_items = n_items;
    ga.counts = a->counts;
    ga.per_req = (uint32_t)per;
    magic_div(per, &ga.div_mul, &ga.div_shift);
    // short fragments go several to a wavefront: all of them where a full fragment is short, else
    // the remainder fragment that ends every request
    const uint64_t full_frag = a->fixed_req_size < a->mtu ? a->fixed_req_size : a->mtu;
    const uint64_t last_frag = a->fixed_req_size - (per - 1) * a->mtu;
    uint32_t small_all = 0, small_last = 0;
    if (!(a->flags & SG_F_NO_SMALL)) {
      small_all = small_lanes(full_frag);
      if (!small_all && last_frag < a->mtu && small_last_pays(per, a->n_req, a->flags, false)) small_last = small_lanes(last_frag);
    }
    ga.per_launch = small_last ? (uint32_t)per - 1 : (uint32_t)per;
    magic_div(ga.per_launch, &ga.lmul, &ga.lshift);
    ga.mtu = a->mtu;
    ga.slot_size = a->ring.slot_size;
    ga.hl = hl0;
    ga.n_slots = a->ring.n_slots;
    ga.n_req = a->n_req;
    ga.frag_len = a->frag_len;
    ga.first = a->req_first;
    ga.offsets_out = packed ? a->offsets_out : nullptr;
    ga.status = sc.status;
    ga.status_flag = sc.flag;
    ga.app = app;
    ga.pieces = pieces_for(a->mtu);
    if (app.n_tensors > 1) ga.n_plan = fill_plan(app, a->fixed_req_size, a->mtu, per, ga.plan);
    uint32_t grid, remap;
    uint64_t waves = (uint64_t)a->n_req * ga.per_launch * ga.pieces;
    if (small_last) {
      // turns of `period` wavefronts: the full fragments of 64 / small_last requests, then their remainders
      const uint32_t per_turn = kWave / small_last;
      ga.period = ga.per_launch * ga.pieces * per_turn + 1;
      magic_div(ga.period, &ga.pmul, &ga.pshift);
      waves = (uint64_t)((a->n_req + per_turn - 1) / per_turn) * ga.period;
      if (waves >= (1u << 27)) return fail(c, SG_E_INVAL, "%llu wavefronts in one call: the limit is 2^27 - 1", (unsigned long long)waves);
    }
    geometry(waves, !(a->flags & SG_F_NO_XCD_REMAP), &grid, &remap);
    ga.opts = (remap ? kOptRemap : 0u) | (app.mirrored ? kOptMirrored : 0u) |
              (app.n_tensors > 1 ? kOptMultiTensor : 0u) | (small_last ? kOptSmallLast : 0u) |
              ((((uintptr_t)a->ring.base | a->ring.slot_size) & 15u) ? 0u : kOptHdrChunk);
    rc = prof_begin(c, 1);
    if (rc != SG_OK) return rc;
    if (small_all) {
      const uint32_t per_wave = kWave / small_all;
      const uint32_t sgrid = (n_items + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
      if (small_all == 16) k_gather_small<16><<<sgrid, kBlock, 0, st>>>(ga);
      else k_gather_small<32><<<sgrid, kBlock, 0, st>>>(ga);
    } else if (small_last == 16) {
      if (ga.pieces > 1) k_gather_rule<true, 16><<<grid, kBlock, 0, st>>>(ga);
      else k_gather_rule<false, 16><<<grid, kBlock, 0, st>>>(ga);
    } else if (small_last == 32) {
      if (ga.pieces > 1) k_gather_rule<true, 32><<<grid, kBlock, 0, st>>>(ga);
      else k_gather_rule<false, 32><<<grid, kBlock, 0, st>>>(ga);
    } else {
      if (ga.pieces > 1) k_gather_rule<true, 0><<<grid, kBlock, 0, st>>>(ga);
      else k_gather_rule<false, 0><<<grid, kBlock, 0, st>>>(ga);
    }
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
    launch_finish(sc, st, packed ? sc.cursor[0] : nullptr, a->fixed_req_size, app.cap, a->n_req, a->counts,
                  a->slot_state, a->n_slot_states, 0, false);
    return finish(c, a->flags);
  }

  PrepArgs p;
  memset(&p, 0, sizeof p);
  p.mode = 0;
  p.n_req = a->n_req;
  p.ring = static_cast<const uint8_t *>(a->ring.base);
  p.n_slots = a->ring.n_slots;
  p.slot_size = a->ring.slot_size;
  p.hl = hdr_len_of(a->ring.hdr_profile);
  p.item_slot = a->frag_slot;
  p.item_len = a->frag_len;
  p.first = a->req_first;
  p.n_items = a->n_frags;
  p.packed = packed;
  p.cap = app.cap;
  p.max_req_bytes = max_req_bytes;
  p.desc = sc.desc;
  p.req_size = sc.req_size;
  p.req_off = sc.req_off;
  p.fixed_size = a->fixed_req_size;
  p.fixed_offsets = p.packed && a->fixed_req_size != 0;
  p.cursor = sc.cursor[0];
  p.next_cursor = sc.next_cursor[0];
  p.offsets_out = packed ? a->offsets_out : nullptr;
  p.counts = a->counts;
  if (sc.desc_gen) {
    p.desc_tag = sc.desc_tag;
    p.gen = ++*sc.desc_gen ? *sc.desc_gen : ++*sc.desc_gen;  // never zero
  }
  p.status = sc.status;
  p.status_flag = sc.flag;
  rc = launch_prep(c, sc, st, p);
  if (rc != SG_OK) return rc;

  // the copy kernel also commits the advanced cursor, so a batch of empty requests still launches it
  if (a->n_frags || packed) {
    GatherArgs ga;
    memset(&ga, 0, sizeof ga);
    ga.desc = sc.desc;
    ga.req_off = sc.req_off;
    ga.ring = p.ring;
    ga.slot_size = p.slot_size;
    ga.hl = p.hl;
    ga.n_items = a->n_frags;
    ga.status = sc.status;
    ga.status_flag = sc.flag;
    if (packed) {
      ga.cursor = sc.cursor[0];
      ga.next_cursor = sc.next_cursor[0];
    }
    ga.counts = a->counts;
    ga.app = app;
    ga.pieces = pieces_for(p.slot_size - p.hl);
    uint32_t grid;
    geometry((uint64_t)(a->n_frags ? a->n_frags : 1u) * ga.pieces, !(a->flags & SG_F_NO_XCD_REMAP), &grid, &ga.remap);
    rc = prof_begin(c, 1);
    if (rc != SG_OK) return rc;
    if (ga.pieces > 1) k_gather<true><<<grid, kBlock, 0, st>>>(ga);
    else k_gather<false><<<grid, kBlock, 0, st>>>(ga);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  launch_finish(sc, st, nullptr, 0, 0, a->n_req, a->counts, a->slot_state, a->n_slot_states, 0, true);
  return finish(c, a->flags);
}

int sg_hip_gather_batch(sg_hip_ctx *c, const sg_gather_args *a)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard g(c->device);
  return gather_impl(c, c->sc, c->stream, a);
}

static int scatter_impl(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const sg_scatter_args *a)
{
  int rc = check_ring(c, a->rx, "rx");
  if (rc != SG_OK) return rc;
  rc = check_ring(c, a->tx, "tx");
  if (rc != SG_OK) return rc;
  if (a->rx.hdr_profile != a->tx.hdr_profile) return fail(c, SG_E_INVAL, "rx and tx rings differ in header profile");
  if (a->n_req == 0) return SG_OK;
  if (a->n_req > sc.max_reqs) return fail(c, SG_E_INVAL, "n_req %u > max_reqs %u", a->n_req, sc.max_reqs);
  if (a->n_frames > sc.max_frames) return fail(c, SG_E_INVAL, "n_frames %u > max_frames %u", a->n_frames, sc.max_frames);
  if (!a->resp_first || (a->n_frames && (!a->tx_slot || (!a->hdr_src_slot && !a->hdr_src_req && !a->hdr_templates))))
    return fail(c, SG_E_INVAL, "null frame tables");
  if ((uintptr_t)a->hdr_templates & 1u) return fail(c, SG_E_INVAL, "hdr_templates must start at an even address");
  const uint32_t hl = hdr_len_of(a->tx.hdr_profile);
  if (a->mtu == 0 || (uint64_t)a->mtu + hl > a->tx.slot_size)
    return fail(c, SG_E_INVAL, "mtu %u + %u header bytes does not fit a %u-byte slot", a->mtu, hl, a->tx.slot_size);
  if ((uint64_t)a->mtu + (hl - 42u) + 28u > 0xffffu) return fail(c, SG_E_INVAL, "mtu %u overflows the IPv4 length field", a->mtu);
  AppDev app;
  uint64_t max_req_bytes;
  rc = check_app(c, a->app, &app, &max_req_bytes);
  if (rc != SG_OK) return rc;
  const bool packed = app.n_tensors == 0;
  if (a->slot_state && a->n_slot_states == 0) return fail(c, SG_E_INVAL, "a slot ring of no slots");
  if (a->slot_state && a->n_req > a->n_slot_states)
    return fail(c, SG_E_INVAL, "%u responses do not fit a ring of %u application slots", a->n_req, a->n_slot_states);

  const bool reuse = (a->flags & SG_F_REUSE_DESC) != 0;
  if (reuse && (!packed || !sc.desc_gen || !*sc.desc_gen))
    return fail(c, SG_E_INVAL, "SG_F_REUSE_DESC needs a packed arena and a descriptor pass of an earlier call on this context");
  const bool fused = a->resp_size == nullptr && !(a->flags & (SG_F_NO_FUSE | SG_F_REUSE_DESC));
  if (fused) {
    if (a->fixed_resp_size == 0 || a->fixed_resp_size > 0xffffffffull)
      return fail(c, SG_E_INVAL, "fixed response size %llu out of range", (unsigned long long)a->fixed_resp_size);
    const uint64_t per = (a->fixed_resp_size + a->mtu - 1) / a->mtu;
    if (a->counts ? per * a->n_req > a->n_frames : per * a->n_req != a->n_frames)
      return fail(c, SG_E_INVAL, "%u responses of %llu bytes at mtu %u are %llu frames, not %u", a->n_req, (unsigned long long)a->fixed_resp_size, a->mtu, (unsigned long long)(per * a->n_req), a->n_frames);
    const uint32_t n_items = (uint32_t)(per * a->n_req);
    if (app.n_tensors == 0 ? a->fixed_resp_size > app.cap : a->fixed_resp_size > max_req_bytes)
      return fail(c, SG_E_INVAL, "response size %llu does not fit its source", (unsigned long long)a->fixed_resp_size);
    ScatterArgs sa;
    memset(&sa, 0, sizeof sa);
    sa.hdr_src_slot = a->hdr_src_slot;
    sa.hdr_templates = a->hdr_templates;
    sa.req_token = a->req_token;
    sa.rx = static_cast<const uint8_t *>(a->rx.base);
    sa.rx_slot_size = a->rx.slot_size;
    sa.rx_n_slots = a->rx.n_slots;
    sa.tx = static_cast<uint8_t *>(a->tx.base);
    sa.tx_slot_size = a->tx.slot_size;
    sa.hl = hl;
    sa.ref64 = a->tx.hdr_profile == SG_HDR_REF64;
    sa.flags = a->flags & 0xfu;
    sa.n_items = n_items;
    sa.n_req = a->n_req;
    sa.counts = a->counts;
    sa.hdr_src_req = a->hdr_templates ? nullptr : a->hdr_src_req;
    sa.status = sc.status;
    sa.status_flag = sc.flag;
    sa.app = app;
    sa.rule.item_slot = a->tx_slot;
    sa.rule.first = a->resp_first;
    sa.rule.size = a->fixed_resp_size;
    sa.rule.mtu = a->mtu;
    sa.rule.per_req = (uint32_t)per;
    sa.rule.per_launch = (uint32_t)per;
    magic_div(per, &sa.rule.div_mul, &sa.rule.div_shift);
    if (n_items >= (1u << 27)) return fail(c, SG_E_INVAL, "%u frames in one call: the limit is 2^27 - 1", n_items);
    sa.rule.n_req = a->n_req;
    sa.rule.n_slots = a->tx.n_slots;
    sa.rule.single_wrap = app.n_tensors == 0 && (uint64_t)a->n_req * a->fixed_resp_size <= app.cap;
    sa.rule.cursor = sc.cursor[1];
    sa.rule.offsets_out = packed ? a->offsets_out : nullptr;
    if (app.n_tensors > 0) sa.n_plan = fill_plan(app, a->fixed_resp_size, a->mtu, per, sa.plan);
    sa.pieces = pieces_for(a->mtu);
    uint32_t grid;
    // short frames go several to a wavefront: all of them where a full frame is short, else the
    // remainder frame that ends every response
    const bool full_csum = (a->flags & SG_F_UDP_CSUM_FULL) != 0;
    const uint64_t full_frame = a->fixed_resp_size < a->mtu ? a->fixed_resp_size : a->mtu;
    const uint64_t last_frame = a->fixed_resp_size - (per - 1) * a->mtu;
    uint32_t small_all = 0, small_last = 0;
    if (!(a->flags & SG_F_NO_SMALL)) {
      small_all = small_lanes(full_frame);
      if (!small_all && last_frame < a->mtu && small_last_pays(per, a->n_req, a->flags, true)) small_last = small_lanes(last_frame);
    }
    rc = prof_begin(c, 2);
    if (rc != SG_OK) return rc;
    if (small_all) {
      launch_scatter_small(st, sa, small_all, n_items, full_csum);
    } else {
      if (small_last) sa.rule.per_launch = (uint32_t)per - 1;
      magic_div(sa.rule.per_launch, &sa.rule.lmul, &sa.rule.lshift);
      const bool defer = csum_in_two_phases(sc, sa.pieces, full_csum);
      sa.csum_part = sc.csum_part;
      sa.csum_valid = sc.csum_valid;
      geometry((uint64_t)a->n_req * sa.rule.per_launch * ((full_csum && !defer) ? 1u : sa.pieces),
               !(a->flags & SG_F_NO_XCD_REMAP), &grid, &sa.remap);
      // (the remainder frames' kernel on a second stream beside this one, forked and joined with
      // events, was measured as well: both kinds of wavefront at once cost the full frames more
      // than the overlap gains, 180 against 172 us on 131072 responses of 1400 + 1400 + 272 bytes)
      launch_scatter<true>(st, sa, grid, full_csum, defer);
      if (small_last) launch_scatter_small(st, sa, small_last, a->n_req, full_csum);
    }
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
    launch_finish(sc, st, packed ? sc.cursor[1] : nullptr, a->fixed_resp_size, app.cap, a->n_req, a->counts,
                  a->slot_state, a->n_slot_states, 1, false);
    return finish(c, a->flags);
  }

  PrepArgs p;
  memset(&p, 0, sizeof p);
  p.mode = 1;
  p.n_req = a->n_req;
  p.n_slots = a->tx.n_slots;
  p.slot_size = a->tx.slot_size;
  p.hl = hl;
  p.mtu = a->mtu;
  p.item_slot = a->tx_slot;
  p.first = a->resp_first;
  p.sizes = a->resp_size;
  p.fixed_size = a->fixed_resp_size;
  p.n_items = a->n_frames;
  p.packed = app.n_tensors == 0;
  p.cap = app.cap;
  p.max_req_bytes = max_req_bytes;
  p.desc = sc.desc;
  p.req_size = sc.req_size;
  p.req_off = sc.req_off;
  p.fixed_offsets = p.packed && a->resp_size == nullptr;
  p.cursor = sc.cursor[1];
  p.next_cursor = sc.next_cursor[1];
  p.offsets_out = packed ? a->offsets_out : nullptr;
  if (!a->hdr_templates) {
    if (a->hdr_src_req) p.hdr_src_req = a->hdr_src_req;
    else p.hdr_src_slot = a->hdr_src_slot;
    p.rx_n_slots = a->rx.n_slots;
  }
  p.counts = a->counts;
  if (sc.desc_gen && !reuse) {
    p.desc_tag = sc.desc_tag;
    p.gen = ++*sc.desc_gen ? *sc.desc_gen : ++*sc.desc_gen;
  }
  p.status = sc.status;
  p.status_flag = sc.flag;
  if (!reuse) {
    rc = launch_prep(c, sc, st, p);
    if (rc != SG_OK) return rc;
  }

  if (a->n_frames || packed) {
    ScatterArgs sa;
    memset(&sa, 0, sizeof sa);
    sa.desc = sc.desc;
    sa.req_off = sc.req_off;
    sa.first = a->resp_first;
    sa.hdr_src_slot = a->hdr_src_slot;
    sa.hdr_templates = a->hdr_templates;
    sa.req_token = a->req_token;
    sa.rx = static_cast<const uint8_t *>(a->rx.base);
    sa.rx_slot_size = a->rx.slot_size;
    sa.rx_n_slots = a->rx.n_slots;
    sa.tx = static_cast<uint8_t *>(a->tx.base);
    sa.tx_slot_size = a->tx.slot_size;
    sa.hl = hl;
    sa.ref64 = a->tx.hdr_profile == SG_HDR_REF64;
    sa.flags = a->flags & 0xfu;
    sa.n_items = a->n_frames;
    sa.n_req = a->n_req;
    sa.counts = a->counts;
    sa.hdr_src_req = a->hdr_templates ? nullptr : a->hdr_src_req;
    sa.status = sc.status;
    sa.status_flag = sc.flag;
    if (packed) {
      sa.cursor = sc.cursor[1];
      sa.next_cursor = sc.next_cursor[1];
    }
    if (reuse) {
      // the response cursor ends up where the reused descriptors end
      sa.next_cursor = sc.next_cursor[0];
      sa.desc_tag = sc.desc_tag;
      sa.reuse_gen = *sc.desc_gen;
      sa.tx_n_slots = a->tx.n_slots;
      sa.offsets_out = a->offsets_out;
    }
    sa.app = app;
    sa.pieces = pieces_for(a->mtu);
    uint32_t grid;
    const bool full_csum = (a->flags & SG_F_UDP_CSUM_FULL) != 0;
    const bool defer = csum_in_two_phases(sc, sa.pieces, full_csum);
    sa.csum_part = sc.csum_part;
    sa.csum_valid = sc.csum_valid;
    geometry((uint64_t)(a->n_frames ? a->n_frames : 1u) * ((full_csum && !defer) ? 1u : sa.pieces),
             !(a->flags & SG_F_NO_XCD_REMAP), &grid, &sa.remap);
    rc = prof_begin(c, 2);
    if (rc != SG_OK) return rc;
    launch_scatter<false>(st, sa, grid, full_csum, defer);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  launch_finish(sc, st, nullptr, 0, 0, a->n_req, a->counts, a->slot_state, a->n_slot_states, 1, true);
  return finish(c, a->flags);
}

int sg_hip_scatter_batch(sg_hip_ctx *c, const sg_scatter_args *a)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard g(c->device);
  return scatter_impl(c, c->sc, c->stream, a);
}

// ---- allocation-free gather ---------------------------------------------------

namespace {
constexpr int kStaticMaxDevices = 64;
std::mutex g_static_mu;
uint8_t *g_static_ptr[kStaticMaxDevices];  // device address of `scratch` on each GPU, once asked for

// The device address of this GPU's copy of the static array (every GPU holds
// its own copy at its own address).  The device must be current.
int static_scratch_of(int device, uint8_t **out)
{
  if (device < 0 || device >= kStaticMaxDevices) return fail(nullptr, SG_E_INVAL, "device %d out of range", device);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[device]) {
    uint8_t *p = nullptr;
    HIP_TRY(nullptr, hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(nullptr, SG_E_HIP, "hipGetSymbolAddress returned a null address on device %d", device);
    g_static_ptr[device] = p;
  }
  *out = g_static_ptr[device];
  return SG_OK;
}
}  // namespace

int sg_hip_gather_batch_static(int device_id, void *stream, const sg_gather_args *a, uint64_t *cursor,
                               uint32_t *status)
{
  if (!a) return fail(nullptr, SG_E_INVAL, "null argument");
  DeviceGuard g(device_id);
  if (!g.ok) return fail(nullptr, SG_E_HIP, "cannot select device %d", device_id);
  uint8_t *base = nullptr;
  int rc = static_scratch_of(device_id, &base);
  if (rc != SG_OK) return rc;
  if (a->n_req > SG_STATIC_MAX_REQS || a->n_frags > SG_STATIC_MAX_FRAMES)
    return fail(nullptr, SG_E_INVAL,
                "%u requests in %u fragments: the allocation-free gather takes at most %u requests in %u fragments",
                a->n_req, a->n_frags, (unsigned)SG_STATIC_MAX_REQS, (unsigned)SG_STATIC_MAX_FRAMES);
  hipStream_t st = static_cast<hipStream_t>(stream);
  Scratch sc;
  sc.max_reqs = SG_STATIC_MAX_REQS;
  sc.max_frames = SG_STATIC_MAX_FRAMES;
  uint8_t *m = base;
  sc.desc = reinterpret_cast<u32x4 *>(m); m += kStaticDesc;
  sc.req_size = reinterpret_cast<uint64_t *>(m); m += kStaticReq;
  sc.req_off = reinterpret_cast<uint64_t *>(m); m += kStaticReq;
  sc.tile_tot = reinterpret_cast<uint64_t *>(m); m += kStaticTile;
  uint64_t *w64 = reinterpret_cast<uint64_t *>(m);      // [0] the array's own cursor, [1] unused, [2] staged cursor
  uint32_t *w32 = reinterpret_cast<uint32_t *>(m + 64);  // [0] the array's own status word, [1] refusal flag
  sc.cursor[0] = cursor ? cursor : w64;
  sc.cursor[1] = nullptr;
  sc.next_cursor[0] = w64 + 2;
  sc.next_cursor[1] = nullptr;
  sc.status = status ? status : w32;
  sc.flag = w32 + 1;
  sc.slot_idx[0] = w32 + 2;  // the array's own producer index, for callers that pass a slot ring
  sc.slot_idx[1] = w32 + 3;
  // descriptors, request totals, offsets and the staged cursor are written by this call's own
  // kernels before they are read; the array's own status word would carry the last call's refusals
  if (!status) k_zero_words<<<1, kBlock, 0, st>>>(w32, 2);
  return gather_impl(nullptr, sc, st, a);
}

// ---- reassembly ----------------------------------------------------------------

namespace {

uint32_t pow2_at_least(uint64_t v)
{
  uint32_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

// Carves the reassembly state out of c->ra_mem (allocating it first where needed).
int ra_state(sg_hip_ctx *c, RaArgs *r, bool *fresh)
{
  const uint32_t n_max = c->max_frames;
  const uint32_t cells = pow2_at_least(4ull * c->max_reqs < 2 * kRaBucket ? 2 * kRaBucket : 4ull * c->max_reqs);
  const uint32_t records = pow2_at_least(c->max_reqs);
  const size_t n_blk = (n_max + kRaBlock - 1) / kRaBlock + 1;
  const size_t bytes = (size_t)cells * (8 + 8 + 4 * 4) + (size_t)records * SG_MAX_BI_SIZE * 8 + (size_t)records * 4 +
                       kRaWords * 4 + (size_t)n_max * (3 * 4 + 8) + n_blk * 8 + 256;
  *fresh = false;
  if (!c->ra_mem) {
    // the small allocation first: a context never holds the state without its pinned counts
    if (!c->h_counts) {
      HIP_TRY(c, hipHostMalloc((void **)&c->h_counts, 4 * sizeof(uint32_t), hipHostMallocDefault));
      memset(c->h_counts, 0, 4 * sizeof(uint32_t));
    }
    HIP_TRY(c, hipMalloc(&c->ra_mem, bytes));
    c->ra_cells = cells;
    c->ra_records = records;
    *fresh = true;
  }
  memset(r, 0, sizeof *r);
  uint8_t *m = static_cast<uint8_t *>(c->ra_mem);
  r->keys = reinterpret_cast<unsigned long long *>(m); m += (size_t)cells * 8;
  r->acc = reinterpret_cast<unsigned long long *>(m); m += (size_t)cells * 8;
  r->tab = reinterpret_cast<unsigned long long *>(m); m += (size_t)records * SG_MAX_BI_SIZE * 8;
  r->arr_pack = reinterpret_cast<unsigned long long *>(m); m += (size_t)n_max * 8;
  r->blk = reinterpret_cast<unsigned long long *>(m); m += n_blk * 8;
  r->want = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->last = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->rec = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->seen = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->free_ring = reinterpret_cast<uint32_t *>(m); m += (size_t)records * 4;
  r->words = reinterpret_cast<uint32_t *>(m); m += kRaWords * 4;
  r->arr_cell = reinterpret_cast<uint32_t *>(m); m += (size_t)n_max * 4;
  r->arr_len = reinterpret_cast<uint32_t *>(m); m += (size_t)n_max * 4;
  r->arr_fidx = reinterpret_cast<uint32_t *>(m);
  r->bmask = cells / kRaBucket - 1;
  r->rmask = records - 1;
  r->counts_host = c->h_counts;
  r->status = c->status;
  r->status_flag = c->h_flag;
  return SG_OK;
}

void ra_launch_reset(sg_hip_ctx *c, const RaArgs &r)
{
  const size_t items = (size_t)c->ra_records * SG_MAX_BI_SIZE > c->ra_cells ? (size_t)c->ra_records * SG_MAX_BI_SIZE
                                                                            : c->ra_cells;
  k_ra_reset<<<(uint32_t)((items + 255) / 256), 256, 0, c->stream>>>(r, c->ra_cells, c->ra_records);
}

}  // namespace

int sg_hip_reassemble_reset(sg_hip_ctx *c)
{
  if (!c) return SG_E_INVAL;
  DeviceGuard g(c->device);
  RaArgs r;
  bool fresh;
  int rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  ra_launch_reset(c, r);
  return finish(c, 0);
}

int sg_hip_reassemble_evict(sg_hip_ctx *c, uint32_t max_age_calls, uint32_t *n_evicted_out)
{
  if (!c) return SG_E_INVAL;
  if (n_evicted_out) *n_evicted_out = 0;
  if (!c->ra_mem) return SG_OK;  // nothing has come in yet
  DeviceGuard g(c->device);
  RaArgs r;
  bool fresh;
  int rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  k_zero_words<<<1, kBlock, 0, c->stream>>>(r.words + kRaEvicted, 1);
  k_ra_evict<<<(c->ra_cells + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(r, c->ra_cells, max_age_calls);
  rc = finish(c, 0);
  if (rc != SG_OK) return rc;
  uint32_t n = 0;
  HIP_TRY(c, hipMemcpy(&n, r.words + kRaEvicted, sizeof n, hipMemcpyDeviceToHost));
  if (n_evicted_out) *n_evicted_out = n;
  return SG_OK;
}

int sg_hip_reassemble(sg_hip_ctx *c, const sg_reassemble_args *a, uint32_t *counts_host_out)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  int rc = check_ring(c, a->ring, "rx");
  if (rc != SG_OK) return rc;
  if (counts_host_out) memset(counts_host_out, 0, 4 * sizeof(uint32_t));
  if (a->n_arrivals > c->max_frames) return fail(c, SG_E_INVAL, "n_arrivals %u > max_frames %u of this context", a->n_arrivals, c->max_frames);
  if ((a->n_arrivals && !a->arrivals) || !a->frag_slot || !a->frag_len || !a->req_first) return fail(c, SG_E_INVAL, "null tables");
  const bool ref64 = a->ring.hdr_profile == SG_HDR_REF64;
  if (ref64 && (!a->len_nic || !a->req_size)) return fail(c, SG_E_INVAL, "REF64 headers need len_nic and the server-wide request size");
  DeviceGuard g(c->device);

  RaArgs r;
  bool fresh;
  rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  if (fresh) ra_launch_reset(c, r);
  r.ring = static_cast<const uint8_t *>(a->ring.base);
  r.n_slots = a->ring.n_slots;
  r.slot_size = a->ring.slot_size;
  r.ref64 = ref64;
  r.n = a->n_arrivals;
  r.n_dev = a->n_arrivals_dev;
  r.arrivals = a->arrivals;
  r.len_nic = a->len_nic;
  r.req_size = a->req_size;
  r.max_req = c->max_reqs;
  r.max_frag = c->max_frames;
  r.n_blocks = (a->n_arrivals + kRaBlock - 1) / kRaBlock;
  r.frag_slot = a->frag_slot;
  r.frag_len = a->frag_len;
  r.req_first = a->req_first;
  r.req_token = a->req_token;
  r.req_hdr_slot = a->req_hdr_slot;
  r.counts_out = a->counts_out;

  const uint32_t g_take = (a->n_arrivals + kRaTakeBlock - 1) / kRaTakeBlock;
  rc = prof_begin(c, 5);
  if (rc != SG_OK) return rc;
  if (a->n_arrivals <= (uint32_t)kRaTakeBlock) {
    // a NIC burst (an empty one still leaves its counts): one workgroup, one launch
    k_ra_burst<<<1, kRaTakeBlock, 0, c->stream>>>(r);
  } else {
    k_ra_insert<<<g_take, kRaTakeBlock, 0, c->stream>>>(r);
    k_ra_flag<<<r.n_blocks, kRaBlock, 0, c->stream>>>(r);
    k_ra_scan<<<1, kRaBlock, 0, c->stream>>>(r);
    k_ra_emit<<<g_take, kRaTakeBlock, 0, c->stream>>>(r);
  }
  rc = prof_end(c);
  if (rc != SG_OK) return rc;
  rc = finish(c, a->flags);
  if (rc != SG_OK || (a->flags & SG_F_ASYNC)) return rc;
  if (counts_host_out) memcpy(counts_host_out, c->h_counts, 4 * sizeof(uint32_t));
  return SG_OK;
}

}  // extern "C"
