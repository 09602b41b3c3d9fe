// sg_kernels_prep.h -- the descriptor pass of the gfx950 scatter-gather engine:
// what a batch looks like to the kernels (AppDev, PrepArgs), the kernels that
// turn the fragment tables of a batch into 16-byte run descriptors (k_prep_*)
// and the scans of the request totals through the bump-ring cursor
// (k_req_scan*).  A part of sg_hip.hip's translation unit, included there and
// nowhere else.
#pragma once

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

// words of a descriptor tag
constexpr uint32_t kTagGen = 0, kTagReqs = 1, kTagItems = 2, kTagSlotSize = 3, kTagArena = 4, kTagCap = 6, kTagWords = 8;

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
  // The plain word of the bump-ring cursor.  The descriptor pass only reads it
  // and leaves the advanced value in *next_cursor; the copy kernel of the same
  // call, which does not read the cursor, commits it.
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
  // (SG_F_REUSE_DESC): desc_tag = {gen, requests, items, slot size the lengths were held
  // against, arena base, arena capacity} (kTag*, eight 32-bit words).
  uint32_t *desc_tag;
  uint32_t gen;
  uint64_t arena_base;
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
    a.desc_tag[kTagGen] = a.gen;
    a.desc_tag[kTagReqs] = a.n_req;
    a.desc_tag[kTagItems] = a.n_items;
    a.desc_tag[kTagSlotSize] = a.slot_size;
    a.desc_tag[kTagArena] = (uint32_t)a.arena_base;
    a.desc_tag[kTagArena + 1] = (uint32_t)(a.arena_base >> 32);
    a.desc_tag[kTagCap] = (uint32_t)a.cap;
    a.desc_tag[kTagCap + 1] = (uint32_t)(a.cap >> 32);
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

}  // namespace
