// sg_kernels_reassemble.h -- sorting a burst of arrivals into requests on the
// device (k_ra_*).  A part of sg_hip.hip's translation unit, included there,
// after sg_kernels_prep.h, and nowhere else.
#pragma once

#include "sg_device.h"

#include "sg_kernels_prep.h"

namespace {

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
  uint32_t blk_size;  // threads per workgroup of k_ra_flag: one entry of blk each
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
// The same steps in workgroups of kRaSmallBlock threads, for a call that runs beside a long copy
// kernel of another stream: a workgroup of sixteen wavefronts finds no room on a chip that such a
// kernel keeps full (it needs sixteen free slots on one CU at once) and waits until that kernel
// ends; one of four wavefronts takes the slots the copy's own workgroups leave.  Four times the
// additions to the ring words, which is why this is not the form of a call that runs alone.
constexpr int kRaSmallBlock = 256;
template <int B>
__device__ __forceinline__ uint32_t ra_block_take(uint32_t *word, uint32_t n_wave, uint32_t *lds)
{
  constexpr uint32_t kWaves = B / kWave;
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
template <int B>
__device__ __forceinline__ void ra_open_cells(const RaArgs &a, bool claimed, uint32_t cell, uint32_t lane, uint32_t *lds)
{
  const unsigned long long cl = __ballot(claimed);
  const uint32_t base = ra_block_take<B>(&a.words[kRaHead], (uint32_t)__popcll(cl), lds);
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

// What a thread knows of its arrival from one step to the next.  The four-kernel form keeps it in
// device memory (arr_cell / arr_len / arr_fidx / arr_pack); a burst handled by one workgroup keeps
// it in registers: every thread only ever reads its own entries, and a store followed by a load of
// the same word is a memory round trip the burst's latency is made of.
struct RaMine {
  uint32_t slot = 0, cell = kRaNoCell, len = 0, fidx = 0;
  unsigned long long pack = 0;
};

template <bool FUSED, int B>
__device__ __forceinline__ void ra_insert_step(const RaArgs &a, uint32_t i, uint32_t *take, RaMine &mine)
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
    mine.slot = slot;
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
  ra_open_cells<B>(a, opened != kRaNoCell, opened, lane, take);
  mine.cell = cell;
  mine.len = len;
  mine.fidx = fidx;
  if (in_range) {
    if (!FUSED) {
      a.arr_cell[i] = cell;
      a.arr_len[i] = len;
      a.arr_fidx[i] = fidx;
    }
    if (cell == kRaNoCell && token != 0) refuse(a.status, a.status_flag, kStPoolFull);  // bucket full
  }
  // arrivals that belong to no request: token 0, refused, no room
  const unsigned long long lost = __ballot(in_range && cell == kRaNoCell);
  if (lane == 0 && lost) atomicAdd(&a.words[kRaDropped], (uint32_t)__popcll(lost));
}

template <int B>
__global__ __launch_bounds__(B) void k_ra_insert(RaArgs a)
{
  __shared__ uint32_t take[B / kWave + 1];
  RaMine mine;
  ra_insert_step<false, B>(a, blockIdx.x * B + threadIdx.x, take, mine);
}

__device__ __forceinline__ bool ra_complete(const RaArgs &a, uint32_t cell, unsigned long long acc)
{
  return a.ref64 ? ra_bytes(acc) == a.req_size : ra_cnt(acc) == a.want[cell];
}

// Returns the workgroup's packed (requests, fragments) total.
template <bool FUSED, int B>
__device__ __forceinline__ uint64_t ra_flag_step(const RaArgs &a, uint32_t i, uint64_t *wave_tot, RaMine &mine)
{
  const uint32_t n = ra_n(a);
  unsigned long long pack = 0;
  if (i < n) {
    const uint32_t cell = FUSED ? mine.cell : a.arr_cell[i];
    const uint32_t r = cell != kRaNoCell ? a.rec[cell] : kRaNoRec;
    if (r != kRaNoRec) {
      const uint32_t fidx = FUSED ? mine.fidx : a.arr_fidx[i];
      if (fidx < SG_MAX_BI_SIZE) {
        // rr_emplace_mbuf: the entry goes where its sequence number says
        a.tab[(size_t)r * SG_MAX_BI_SIZE + fidx] =
            (unsigned long long)(FUSED ? mine.slot : a.arrivals[i]) | ((unsigned long long)(FUSED ? mine.len : a.arr_len[i]) << 32);
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
  const uint64_t ex = block_exclusive_scan<B>(pack, wave_tot, &tot);
  mine.pack = pack ? (ex | (1ull << 63)) : 0;  // top bit: "a request completes here"
  if (!FUSED && i < n) a.arr_pack[i] = mine.pack;
  return tot;
}

template <int B>
__global__ __launch_bounds__(B) void k_ra_flag(RaArgs a)
{
  __shared__ uint64_t wave_tot[B / kWave];
  RaMine mine;
  const uint64_t tot = ra_flag_step<false, B>(a, blockIdx.x * B + threadIdx.x, wave_tot, mine);
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

// B: this kernel's own workgroup size; a.blk_size: that of the k_ra_flag before it (a total per workgroup).
template <int B>
__global__ __launch_bounds__(B) void k_ra_scan(RaArgs a)
{
  __shared__ uint64_t wave_tot[B / kWave];
  const uint32_t n = ra_n(a);
  const uint32_t n_blocks = (n + a.blk_size - 1) / a.blk_size;
  uint64_t run = 0;
  for (uint32_t base = 0; base < n_blocks; base += B) {
    const uint32_t b = base + threadIdx.x;
    const uint64_t v = b < n_blocks ? a.blk[b] : 0;
    uint64_t tot;
    const uint64_t ex = block_exclusive_scan<B>(v, wave_tot, &tot);
    if (b < n_blocks) a.blk[b] = run + ex;
    run += tot;
  }
  if (threadIdx.x == 0) (void)ra_scan_finish<false>(a, run);
}

// The wavefront of a completing arrival hands the request over: its record goes
// into the output tables in sequence order, the record is emptied and returned
// to the free ring, the cell is emptied.  The request's rank and first fragment
// index hang on that arrival (arr_pack there plus its workgroup's scanned total).
template <bool FUSED, int B>
__device__ __forceinline__ void ra_emit_step(const RaArgs &a, uint32_t i, uint32_t *take, bool overflow, const RaMine &mine)
{
  const uint32_t n = ra_n(a);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t cell = kRaNoCell;
  unsigned long long v = 0;
  bool completes = false;
  if (i < n) {
    cell = FUSED ? mine.cell : a.arr_cell[i];
    const unsigned long long p = FUSED ? mine.pack : a.arr_pack[i];
    completes = cell != kRaNoCell && (p >> 63) && !overflow;
    if (completes) v = (p & ~(1ull << 63)) + (FUSED ? 0ull : a.blk[i / B]);  // one workgroup: nothing before it
    // the position of a request's last arrival counts per call
    if (cell != kRaNoCell && !completes) a.last[cell] = 0;
  }
  unsigned long long todo = __ballot(completes);
  // reap_rr for all of this workgroup's requests: one addition to the ring's tail
  const uint32_t tail0 = ra_block_take<B>(&a.words[kRaTail], (uint32_t)__popcll(todo), take);
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

template <int B>
__global__ __launch_bounds__(B) void k_ra_emit(RaArgs a)
{
  __shared__ uint32_t take[B / kWave + 1];
  ra_emit_step<false, B>(a, blockIdx.x * B + threadIdx.x, take, a.words[kRaOverflow] != 0, RaMine());
}

// A burst of at most kRaTakeBlock arrivals: the four steps by one workgroup in one launch.
static_assert(kRaTakeBlock == kRaBlock, "one workgroup size for all steps of a burst");
__global__ __launch_bounds__(kRaTakeBlock) void k_ra_burst(RaArgs a)
{
  __shared__ uint32_t take[kRaTakeBlock / kWave + 1];
  __shared__ uint64_t wave_tot[kRaBlock / kWave];
  __shared__ uint32_t overflow;
  const uint32_t i = threadIdx.x;
  RaMine mine;
  ra_insert_step<true, kRaTakeBlock>(a, i, take, mine);
  __syncthreads();
  const uint64_t tot = ra_flag_step<true, kRaBlock>(a, i, wave_tot, mine);
  if (threadIdx.x == 0) overflow = ra_scan_finish<true>(a, tot);
  __syncthreads();
  ra_emit_step<true, kRaTakeBlock>(a, i, take, overflow != 0, mine);
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

}  // namespace
