// sg_kernels_copy.h -- the kernels that move bytes: ring slots -> tensors
// (k_gather, k_gather_rule, k_gather_small), tensors -> TX slots with the
// response headers and checksums (k_scatter, k_scatter_small, k_udp_finish),
// the tail of a call (k_finish) and the per-request entry points' kernels
// (k_copy_runs, k_swap_hdrs).  A part of sg_hip.hip's translation unit,
// included there, after sg_kernels_prep.h, and nowhere else.
#pragma once

#include "sg_device.h"

#include "sg_kernels_prep.h"

namespace {

// ---------------------------------------------------------------------------
// gather / scatter
// ---------------------------------------------------------------------------

// Which item a wavefront works on.  Workgroups are dealt round-robin to the
// eight XCDs, each with its own L2.  Runs of kXcdRun consecutive workgroups'
// worth of items are given to one XCD, so that neighbouring fragment runs --
// which share the cache lines at their common destination boundary -- meet in
// one L2, while all XCDs still walk the same region of memory together.
constexpr uint32_t kXcdRun = 32;
__device__ __forceinline__ uint32_t item_of_wave(bool remap, uint32_t block)
{
  uint32_t g = block;
  if (remap) {
    const uint32_t xcd = g % kXcds, k = g / kXcds;
    g = ((k / kXcdRun) * kXcds + xcd) * kXcdRun + (k % kXcdRun);
  }
  return __builtin_amdgcn_readfirstlane(g * kWavesPerBlock + threadIdx.x / kWave);
}

// Behind a call: a one-workgroup kernel that publishes application slot states
// where the caller keeps a slot ring (they may only change once the copy kernel
// is through), and advances the cursor for the calls whose copy kernel does not
// do that itself: a call that publishes slot states, and every call of the
// allocation-free entry point (its cursor is a plain word).  (Letting the
// wavefronts of the copy kernel count themselves out with atomics so that the
// last one may do this work was built and measured: one returning atomic per
// workgroup costs the 32-batch gather 4 to 11 % -- the wavefront that waits for
// its ticket holds its registers that much longer.)
struct FinishArgs {
  uint64_t *cursor;       // advanced by n_req * size modulo cap; nullptr: nothing to advance
  uint32_t cursor_cells;  // the cursor is a context's pair of cells, not a plain word
  uint32_t pad;
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
    const uint64_t c = cursor_get(a.cursor, a.cursor_cells != 0);
    cursor_put(a.cursor, a.cursor_cells != 0, (c % a.cap + ((uint64_t)n * a.size) % a.cap) % a.cap);
  }
  // A call that refused part of its input publishes no slot states and leaves the ring index: a
  // worker that polls the words must not be handed a request with a hole in it.  (The cursor of a
  // call without a descriptor pass has moved all the same, as documented.)
  if (a.state && !refused) {
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
  uint32_t call_seq;            // ADV: the context's count of calls, part of the launch's stamp
  // The plain cursor word.  In the self-advancing kernels (ADV) it is a context's, the live value
  // is in the cells that word belongs to, and the launch writes the successor (it is the call's
  // last kernel that reads the cursor; no k_finish follows).
  uint64_t *cursor;
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
  uint32_t cursor_cells;        // the cursor is a context's pair of cells, not a plain word
  uint32_t cursor_pad;
  AppDev app;
};

// Descriptor of item `item` from the rule; publishes the request offset and, on
// the batch's last item, the advanced cursor.  Returns status bits.
// `writer`: this thread is the one of the launch that advances a self-advancing cursor (ADV).
template <bool ADV>
__device__ __forceinline__ uint32_t rule_desc(const RuleArgs &g, const AppDev &app, uint32_t item,
                                              uint32_t n_items, uint32_t n_req, uint32_t lane, uint32_t *slot,
                                              uint32_t *len, uint32_t *off, uint32_t *r,
                                              uint32_t *i, uint64_t *req_off, bool writer)
{
  uint32_t bad = 0;
  *r = (uint32_t)(((uint64_t)item * g.div_mul) >> g.div_shift);  // item / per_req
  *i = item - *r * g.per_req;
  // the three table reads are independent: asked for together
  *slot = sload_here(g.item_slot + item);
  const uint32_t first_r = sload_here(g.first + *r);
  uint64_t c0 = app.n_tensors == 0 ? sload_here(g.cursor) : 0;
  uint64_t cur_stamp = 0;
  uint32_t cur_live = 0;
  if (ADV && app.n_tensors == 0) c0 = cursor_take(g.cursor - kCurPlain, g.call_seq, &cur_live, &cur_stamp);
  *off = *i * g.mtu;
  const uint64_t rem = g.size - *off;
  *len = (uint32_t)(rem <= g.mtu ? rem : g.mtu);
  if (*slot >= g.n_slots) bad |= kStBadSlot;
  if (*i == 0 && first_r != item) bad |= kStBadTable;
  *req_off = 0;
  if (app.n_tensors == 0) {
    if (c0 >= app.cap) c0 %= app.cap;  // only after a set_cursor beyond the capacity
    // the successor depends on the cursor, the size and the count only: it is out before a bad item is dropped
    if (ADV && writer) cursor_advance(g.cursor - kCurPlain, g.call_seq, cur_live, cur_stamp, cursor_bump(c0, n_req, g.size, app.cap));
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
  const uint32_t w = item_of_wave(remap != 0, blockIdx.x);
  const uint32_t item = LONG ? w / pieces : w;
  const uint32_t piece = LONG ? w - item * pieces : 0;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  // this kernel does not read the cursor: the value the descriptor pass left is committed here
  // (a batch of no requests at all has left none)
  if (w == 0 && lane == 0 && a.cursor && !sload(status) && (!counts || sload(counts)))
    cursor_put(a.cursor, a.cursor_cells != 0, sload(a.next_cursor));
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
struct alignas(64) GatherRuleArgs {
  // hot: what a wavefront needs before its first payload load
  const uint8_t *ring;
  const uint32_t *frag_slot;
  uint8_t *dst;               // arena (packed) or the tensor (one tensor-major buffer)
  uint64_t *cursor;           // packed only: the plain cursor word (ADV kernels: of a context, whose cells hold the live value)
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
  uint32_t call_seq;  // ADV: the context's count of calls, part of the launch's stamp
  alignas(64) FragPlan plan[kPlanMax];  // an entry is one 8-dword scalar load: inside one cache line
};
constexpr uint32_t kOptRemap = 1u, kOptMirrored = 2u, kOptMultiTensor = 8u;
// slots start at 16-byte aligned addresses: the header's length field can be read as part of
// the aligned chunk at byte 48 (a ring only has to start at an even address)
constexpr uint32_t kOptHdrChunk = 16u;
constexpr uint32_t kOptSmallLast = 32u;  // the last fragment of every request is left to k_gather_small

template <int L, bool ADV>
__device__ __forceinline__ void gather_small_wave(const GatherRuleArgs &a, uint32_t wave, bool may_advance, size_t kernarg_base = 0);

// SMALL: lanes per remainder fragment (16 or 32) when the last fragment of every
// request is short -- the wavefronts behind those of the full fragments then move
// 64 / SMALL remainder fragments each, in the same launch (a launch of their own
// would be all latency: tens of megabytes at most); 0: no such wavefronts.
// ADV: the kernel takes the cursor from a context's cells and advances it itself (no k_finish follows).
// `block`: the workgroup's number among those of this work; `kernarg_base`: where `a` lies in the
// running kernel's argument block (the plan is read through the argument pointer).
template <bool LONG, int SMALL, bool ADV>
__device__ __forceinline__ void gather_rule_body(const GatherRuleArgs &a, uint32_t block, size_t kernarg_base)
{
  const uint8_t *ring = a.ring;
  const uint32_t *frag_slot = a.frag_slot;
  const uint32_t *frag_len = a.frag_len;
  uint8_t *dst = a.dst;
  uint64_t *cursor_in = a.cursor;
  const uint64_t size = a.size, cap = a.cap;
  const uint32_t per_req = a.per_req, mtu = a.mtu, slot_size = a.slot_size;
  const uint32_t hl = a.hl, n_slots = a.n_slots, pieces = a.pieces, opts = a.opts;
  const uint32_t div_mul = a.div_mul, div_shift = a.div_shift;
  const uint32_t *counts = a.counts;
  uint32_t n_items = a.n_items, n_req = a.n_req;
  SG_PIN(ring); SG_PIN(frag_slot); SG_PIN(dst); SG_PIN(cursor_in); SG_PIN(size); SG_PIN(cap);
  SG_PIN(n_items); SG_PIN(per_req); SG_PIN(mtu); SG_PIN(slot_size); SG_PIN(hl); SG_PIN(n_slots);
  SG_PIN(pieces); SG_PIN(opts); SG_PIN(div_mul); SG_PIN(div_shift); SG_PIN(counts); SG_PIN(frag_len);
  if (counts) {
    // counts left on the device by the reassembly: the launch was sized for n_req requests at most
    n_req = dev_count(counts, 0, n_req);
    n_items = n_req * per_req;
  }

  uint32_t w = item_of_wave((opts & kOptRemap) != 0, block);
  const bool first_wave = w == 0;
  const uint32_t pl = a.per_launch;
  if (SMALL) {
    // Wavefronts of the two kinds are dealt in turns: after the period - 1 wavefronts of the full
    // fragments of 64 / SMALL requests comes the one that moves those requests' remainders.  The
    // short-fragment wavefronts are bound by their arithmetic, the others by memory: side by side
    // on a CU they overlap, one kind after the other they would not.
    const uint32_t blk = (uint32_t)(((uint64_t)w * a.pmul) >> a.pshift);
    const uint32_t j = w - blk * a.period;
    if (j == a.period - 1) {
      gather_small_wave<(SMALL ? SMALL : 16), ADV>(a, blk, false, kernarg_base);  // wavefront 0 of the full fragments advances the cursor
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
  // where lengths come from a table (the reference's header carries none), the entry is asked for
  // with the slot's: read at the end, where it is held against the rule, it would lengthen the
  // wavefront's life by a round trip of its own
  const uint32_t tab_len = frag_len ? sload(frag_len + item) : 0u;
  uint64_t c0 = cap ? sload(cursor_in) : 0;
  uint64_t cur_stamp = 0;
  uint32_t cur_live = 0;
  if (ADV && cap) c0 = cursor_take(cursor_in - kCurPlain, a.call_seq, &cur_live, &cur_stamp);
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
    // the successor depends on the cursor, the size and the count only: it is out before a
    // fragment with a bad slot index is dropped
    if (ADV && first_wave && lane == 0)
      cursor_advance(cursor_in - kCurPlain, a.call_seq, cur_live, cur_stamp, cursor_bump(c0, n_req, size, cap));
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
      const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(kernarg_base + offsetof(GatherRuleArgs, plan))) + i);
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
  const bool check_hdr = piece == 0 && frag_len == nullptr;
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
    const bool as_ruled = (check_hdr ? hdr_len : tab_len) == len;
    if (!as_ruled) bad |= kStNotRule;
    if (i == 0 && sload(a.first + r) != item) bad |= kStBadTable;
    if (bad && lane == 0) refuse(a.status, a.status_flag, bad);
  }
}

template <bool LONG, int SMALL, bool ADV>
__global__ __launch_bounds__(kBlock) void k_gather_rule(GatherRuleArgs a)
{
  gather_rule_body<LONG, SMALL, ADV>(a, blockIdx.x, 0);
}

// Gather of SHORT fragments, 64 / L fragments per wavefront (L = 16 or 32 lanes
// per fragment): the rule form of the gather for fragments of a few hundred
// bytes -- every fragment of the call (per_launch == per_req) or the last
// fragment of every request (the remainder; the full fragments then go through
// k_gather_rule).  Addressing is per lane.
template <int L, bool ADV>
__device__ __forceinline__ void gather_small_wave(const GatherRuleArgs &a, uint32_t wave, bool may_advance, size_t kernarg_base)
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
    uint64_t cur_stamp = 0;
    uint32_t cur_live = 0;
    if (ADV) c0 = cursor_take(a.cursor - kCurPlain, a.call_seq, &cur_live, &cur_stamp);
    if (c0 >= a.cap) c0 %= a.cap;  // only after a set_cursor beyond the capacity
    if (ADV && may_advance && wave == 0 && lane == 0)
      cursor_advance(a.cursor - kCurPlain, a.call_seq, cur_live, cur_stamp, cursor_bump(c0, n_req, a.size, a.cap));
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
        const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(kernarg_base + offsetof(GatherRuleArgs, plan))) + (per_req - 1));
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
template <int L, bool ADV>
__global__ __launch_bounds__(kBlock) void k_gather_small(GatherRuleArgs a)
{
  gather_small_wave<L, ADV>(a, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave, true);
}

struct alignas(64) ScatterArgs {
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
  uint32_t cursor_cells;        // the cursor is a context's pair of cells, not a plain word
  uint32_t cursor_pad;
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
  alignas(64) FragPlan plan[kPlanMax];  // an entry is one 8-dword scalar load: inside one cache line
};

// Where the payload of a frame comes from; false: not one contiguous piece.
template <bool FUSED>
__device__ __forceinline__ bool scatter_source(const ScatterArgs &a, uint64_t ro, uint32_t r, uint32_t i,
                                               uint32_t off, uint32_t len, uint8_t **from, size_t kernarg_base)
{
  if (FUSED && a.n_plan) {
    const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(kernarg_base + offsetof(ScatterArgs, plan))) + i);
    *from = reinterpret_cast<uint8_t *>(((uint64_t)fp[1] << 32 | fp[0]) + (uint64_t)r * fp[4]);
    return fp[7] == 0;
  }
  return plain_target(a.app, ro, r, off, len, from);
}

static_assert(offsetof(ScatterArgs, plan) % 64 == 0 && offsetof(GatherRuleArgs, plan) % 64 == 0, "plan entries inside cache lines");
constexpr uint32_t kPartStride = 8;  // words of csum_part per frame: up to 7 sub-runs and the header's share

// LONG: frames longer than kPieceChunks chunks are spread over a.pieces
// wavefronts; piece 0 also writes the header.  With the payload sum
// (FULL_CSUM) the wavefronts of a frame each leave the sum of their bytes
// behind and k_udp_finish writes the field (DEFER, below); where there is no
// room for those sums the frame stays with one wavefront, which walks its
// sub-runs two at a time (more in flight cost registers, hence resident
// wavefronts, and measured slower: 3 at a time +1 %, 5 at a time +8 %).
// (Combining the sums with one returning atomic per wavefront was measured:
// the atomic's round trip at the end of every wavefront's life cost more than
// the second launch.)
// DEFER (long frames with the full UDP checksum): the frame's sub-runs go to
// several wavefronts all the same, each leaving the sum of its bytes behind,
// and k_udp_finish writes the checksum field afterwards.
// ADV (fused only): the kernel takes the cursor from a context's cells and advances it itself.
template <bool FULL_CSUM, bool FUSED, bool LONG, bool DEFER, bool ADV>
__device__ __forceinline__ void scatter_body(const ScatterArgs &a, uint32_t block, size_t kernarg_base)
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
  const uint32_t w = item_of_wave(remap != 0, block);
  const uint32_t pieces = SPLIT ? n_pieces : 1u;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  // descriptor path: this kernel does not read the cursor and commits what the descriptor pass left
  if (!FUSED && a.reuse_gen && n_req) {
    // the caller says these are the items the tagged descriptor pass described: the tag holds that
    // pass's generation and counts, the slot size its lengths were held against, and the arena its
    // offsets lie in.  A call that departs from any of them moves nothing.
    const u32x8 tg = sload(reinterpret_cast<const u32x8 *>(a.desc_tag));
    uint32_t bad = 0;
    if (tg[kTagGen] != a.reuse_gen || tg[kTagReqs] != n_req || tg[kTagItems] != n_items) bad |= kStBadTable;
    if (tg[kTagSlotSize] > tx_slot_size) bad |= kStBadLen;  // lengths were only held against that slot size
    const uint64_t t_base = (uint64_t)tg[kTagArena + 1] << 32 | tg[kTagArena], t_cap = (uint64_t)tg[kTagCap + 1] << 32 | tg[kTagCap];
    if (t_base != (uint64_t)(uintptr_t)a.app.arena || t_cap != a.app.cap) bad |= kStBadSize;  // offsets of another arena
    if (bad) {
      if (w == 0 && lane == 0) refuse(a.status, a.status_flag, bad);
      return;
    }
  }
  if (!FUSED && w == 0 && lane == 0 && a.cursor && !sload(status) && (!counts || sload(counts))) {
    const uint64_t nc = sload(a.next_cursor);
    cursor_put(a.cursor, a.cursor_cells != 0, nc);
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
      if (d[0] >= a.tx_n_slots || d[1] > a.rule.mtu) {  // described for another ring, or cut at another mtu
        if (lane == 0 && piece == 0) refuse(a.status, a.status_flag, d[0] >= a.tx_n_slots ? kStBadSlot : kStBadLen);
        return;
      }
      if (a.offsets_out && item == f0 && lane == 0 && piece == 0) a.offsets_out[r] = ro;
    }
  } else {
    uint32_t slot_i, len, off, i;
    const uint32_t bad = rule_desc<ADV>(a.rule, a.app, item, n_items, n_req, piece == 0 ? lane : 1u, &slot_i, &len,
                                   &off, &r, &i, &ro, w == 0 && lane == 0);
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
    if (d[1] && scatter_source<FUSED>(a, ro, r, item - f0, d[2], d[1], &from, kernarg_base)) {
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
  const bool plain = d[1] != 0 && scatter_source<FUSED>(a, ro, r, item - f0, d[2], d[1], &from, kernarg_base);
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

template <bool FULL_CSUM, bool FUSED, bool LONG, bool DEFER = false, bool ADV = false>
__global__ __launch_bounds__(kBlock) void k_scatter(ScatterArgs a)
{
  scatter_body<FULL_CSUM, FUSED, LONG, DEFER, ADV>(a, blockIdx.x, 0);
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

// Scatter of SHORT frames, 64 / L frames per wavefront (L = 8, 16 or 32 lanes per
// frame): the fused form of k_scatter -- responses of one size cut by the
// fragmenting rule -- for frames of a few hundred bytes, where one wavefront per
// frame spends most of its time on addressing and header arithmetic that 48 of
// its 64 lanes take no part in.  Either every frame of the call (rule.per_launch
// == rule.per_req) or the last frame of every response (the remainder; the full
// frames then go through k_scatter).  Addressing is per lane, the header is two
// 16-bit words per lane, sums are row reductions.
template <int L, bool FULL_CSUM, bool ADV>
__device__ __forceinline__ void scatter_small_wave(const ScatterArgs &a, uint32_t wave, size_t kernarg_base = 0)
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
    uint64_t cur_stamp = 0;
    uint32_t cur_live = 0;
    if (ADV) c0 = cursor_take(a.rule.cursor - kCurPlain, a.rule.call_seq, &cur_live, &cur_stamp);
    if (c0 >= a.app.cap) c0 %= a.app.cap;  // only after a set_cursor beyond the capacity
    if (ADV && wave == 0 && lane == 0)
      cursor_advance(a.rule.cursor - kCurPlain, a.rule.call_seq, cur_live, cur_stamp, cursor_bump(c0, n_req, a.rule.size, a.app.cap));
    uint64_t o = c0 + (uint64_t)r * a.rule.size;
    if (a.rule.single_wrap) o = o >= a.app.cap ? o - a.app.cap : o;
    else o %= a.app.cap;
    ro = o;
  }
  uint8_t *from = nullptr;
  bool plain;
  if (last_only && a.n_plan) {
    // every group has the response's last frame: one plan entry for the wavefront
    const u32x8 fp = sload(reinterpret_cast<const u32x8 *>(kernarg_at(kernarg_base + offsetof(ScatterArgs, plan))) + (per_req - 1));
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
  constexpr int W = L == 8 ? 4 : 2;  // header words per lane
  const SmallHdr<W> sh = small_hdr_fetch<W>(hin, gl, hl, !from_template, live && gl < 32 / W);
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
  small_hdr_finish<L, W>(sh, slot, gl, hf, psum, live);
}

// Every frame of the call is short.
template <int L, bool FULL_CSUM, bool ADV>
__global__ __launch_bounds__(kBlock) void k_scatter_small(ScatterArgs a)
{
  scatter_small_wave<L, FULL_CSUM, ADV>(a, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave);
}

// One pass of the shunter's loop (src/splitrpc_server/p2p_rpc_dpdk_server.cc:117-189) in ONE
// launch: the first s_blocks workgroups scatter the responses that are done (one response size),
// the others gather the requests that became ready (declared rule), each half exactly as the
// kernel of its own would.  Both halves advance their cursors themselves.  For calls that the chip
// holds at once (a batch or two) a launch costs more than the bytes it moves; this halves the
// launches of a step.  The scatter's wavefronts live longest (a header to fetch, rewrite and store
// besides the payload) and are few: their workgroups come first, so that they end with the others,
// not after.  (Larger calls lose by sharing a launch -- 8 resnet50-sized batches 30.2 -> 32.2 us
// per step, 2048 lenet-sized ones 86.4 -> 96.9 us, wherever in the grid the scatter's workgroups
// are put: first, or spread through the gather's in groups of eight, one per XCD -- and are made
// as two calls on a stream each.)
// G_SMALL: the gather's short last fragments go SMALL lanes each (gather_rule_body); S_SMALL: all
// of the scatter's frames are short and go S_SMALL lanes each (scatter_small_wave).
struct alignas(64) ShuntArgs {
  GatherRuleArgs g;
  ScatterArgs s;
  uint32_t s_blocks;
};

template <int G_SMALL, int S_SMALL, bool FULL_CSUM>
__global__ __launch_bounds__(kBlock) void k_shunt(ShuntArgs a)
{
  const uint32_t b = blockIdx.x;
  if (b >= a.s_blocks) {
    gather_rule_body<false, G_SMALL, true>(a.g, b - a.s_blocks, offsetof(ShuntArgs, g));
  } else if (S_SMALL) {
    scatter_small_wave<(S_SMALL ? S_SMALL : 8), FULL_CSUM, true>(a.s, b * kWavesPerBlock + threadIdx.x / kWave, offsetof(ShuntArgs, s));
  } else {
    scatter_body<FULL_CSUM, true, false, false, true>(a.s, b, offsetof(ShuntArgs, s));
  }
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

// Sets `n` 32-bit words to zero (a fill kernel rather than a memset node, so
// that callers may record the launch into a graph).
__global__ __launch_bounds__(kBlock) void k_zero_words(uint32_t *p, uint32_t n)
{
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace
