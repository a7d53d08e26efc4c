// Expert-sorted token alignment (counting sort by expert, padded to blocks).
//
// Replaces moe_align_block_size_kernel + count_and_sort_expert_tokens_kernel of
// the reference (csrc/moe_align_block_size_kernels.cu:140-237).  The reference
// ranks tokens inside an expert's segment with a global atomicAdd, which makes
// the order arbitrary; here the flat index range is cut into contiguous
// segments, one wavefront per segment, and a token's rank is
//     (tokens of its expert in earlier segments)            -- prefix over segments
//   + (tokens of its expert earlier in this segment)        -- running LDS counter
//   + (same-expert lanes below it in the current 64 ids)    -- ballot + popcount
// which is the stable order and needs no global atomics.
//
// Small inputs run as ONE workgroup of 16 wavefronts (histogram, scans and
// scatter in LDS); larger ones as two launches (count, then scan + scatter with
// every workgroup deriving its own prefixes) with the per-segment histograms in
// the caller's workspace; three launches (count / scan / scatter) when the
// tables of the second launch would not fit in LDS.
#include "common.h"
#include "routing_device.h"

namespace {

constexpr int kMaxExperts = 1024;
// Rows the routing + alignment workgroup takes.  One workgroup routes 32 rows of 128 experts side by
// side in about 6 us (one CU's instruction throughput: a row is ~750 instructions), and every further
// 32 rows cost as much again, while the stand-alone router spreads its rows over the whole chip:
// measured on the Qwen3-30B-A3B router (128 experts, top-8), launches included, 14.8 us against
// 17.7 us for the two kernels at 32 rows, 21.0 against 17.6 at 64, 59.7 against 17.2 at 256.
// What it saves at 32 rows is host time only: replayed from a HIP graph the one launch takes 14.7 us
// and the two kernels 13.2 us (they follow each other within about a microsecond).  Spreading the
// routing over several workgroups and letting the last one to finish align (release fence, arrival
// counter, acquire fence) cost 4.5 us more than the two kernels from 64 to 256 rows.
constexpr int kRouteAlignMaxTokens = 32;
constexpr int kScanThreads = 1024;              // one thread per expert in the scans
constexpr int kScanWaves = kScanThreads / kWave;
constexpr int kSegLen = 512;                    // ids per wavefront segment, large path
constexpr int64_t kSmallNumel = 16384;          // at or below: single-workgroup path ...
constexpr int kSmallMaxExperts = 512;           // ... when its LDS histograms fit in 64 KB

__device__ __forceinline__ int load_id(const void* ids, int dtype, int64_t i) {
  switch (dtype) {
    case MOE_ID_I32: return static_cast<const int32_t*>(ids)[i];
    case MOE_ID_I64: {
      int64_t v = static_cast<const int64_t*>(ids)[i];
      return (v < 0 || v > INT32_MAX) ? -1 : static_cast<int>(v);
    }
    case MOE_ID_I16: return static_cast<const int16_t*>(ids)[i];
    case MOE_ID_I8: return static_cast<const int8_t*>(ids)[i];
    default: return static_cast<const uint8_t*>(ids)[i];
  }
}

// Lanes of the wavefront whose (valid) id equals this lane's id.
__device__ __forceinline__ uint64_t same_id_lanes(int id, bool valid, int id_bits) {
  uint64_t m = __ballot(valid);
  for (int b = 0; b < id_bits; ++b) {
    const bool bit = (id >> b) & 1;
    const uint64_t bal = __ballot(bit);
    m &= bit ? bal : ~bal;
  }
  return m;
}

__device__ __forceinline__ uint64_t lanes_below(int lane) { return (1ull << lane) - 1ull; }

// Exclusive prefix sum of one int per thread over a kScanThreads workgroup.
// `wave_tot` is LDS scratch of kScanWaves + 1 ints; slot kScanWaves receives
// the grand total.  Contains workgroup barriers.
__device__ int block_exclusive_scan(int v, volatile int* wave_tot) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  int inc = v;
#pragma unroll
  for (int d = 1; d < kWave; d *= 2) {
    int o = __shfl_up(inc, d, kWave);
    if (lane >= d) inc += o;
  }
  if (lane == kWave - 1) wave_tot[wave] = inc;
  __syncthreads();
  if (wave == 0) {
    int w = lane < kScanWaves ? wave_tot[lane] : 0;
    int winc = w;
#pragma unroll
    for (int d = 1; d < kScanWaves; d *= 2) {
      int o = __shfl_up(winc, d, kWave);
      if (lane >= d) winc += o;
    }
    if (lane < kScanWaves) wave_tot[lane] = winc - w;
    if (lane == kScanWaves - 1) wave_tot[kScanWaves] = winc;
  }
  __syncthreads();
  return inc - v + wave_tot[wave];
}

// After `cum[0..E]` (LDS) holds the padded exclusive prefix and `tot[e]` the
// raw counts: writes expert_ids, num_tokens_post_pad and every padding slot
// of sorted_token_ids.  Called by all kScanThreads threads.
__device__ void write_blocks_and_padding(const volatile int* cum, const volatile int* tot, int E,
                                         int BM, int numel, int32_t* sorted_ids,
                                         int64_t sorted_cap, int32_t* expert_ids,
                                         int64_t expert_cap, int32_t* num_post_pad) {
  const int total = cum[E];
  if (threadIdx.x == 0) *num_post_pad = total;
  const int used_blocks = total / BM;
  for (int b = threadIdx.x; b < used_blocks; b += kScanThreads) {
    const int pos = b * BM;
    // first j in [1, E] with cum[j] > pos; the block belongs to expert j - 1
    int lo = 1, hi = E;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (cum[mid] > pos) hi = mid; else lo = mid + 1;
    }
    expert_ids[b] = lo - 1;
  }
  for (int64_t b = used_blocks + threadIdx.x; b < expert_cap; b += kScanThreads) expert_ids[b] = 0;
  // padding inside each expert's last block: one wavefront per expert
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  for (int e = wave; e < E; e += kScanWaves) {
    const int beg = cum[e] + tot[e], end = cum[e + 1];
    for (int p = beg + lane; p < end; p += kWave) sorted_ids[p] = numel;
  }
  for (int64_t p = total + threadIdx.x; p < sorted_cap; p += kScanThreads) sorted_ids[p] = numel;
}

// Walks ids [beg, end) in order, 64 at a time, and writes each flat index to
// its slot.  `run[e]` (LDS, private to this wavefront) holds the next free
// slot of expert e and is advanced by the lowest lane of every same-id group.
__device__ __forceinline__ void scatter_segment(const void* ids, int dtype, int64_t beg,
                                                int64_t end, int E, int id_bits,
                                                volatile int* run, int32_t* sorted_ids) {
  const int lane = threadIdx.x % kWave;
  auto place = [&](int64_t i, int id) {
    const bool valid = id >= 0 && id < E;
    const uint64_t grp = same_id_lanes(id, valid, id_bits);
    if (valid) {
      const int below = __popcll(grp & lanes_below(lane));
      const int slot = run[id] + below;
      sorted_ids[slot] = static_cast<int32_t>(i);
      if (below == 0) run[id] = slot + __popcll(grp);
    }
  };
  // the ids of up to eight steps are fetched at once: loaded step by step, every
  // step would wait out one memory latency before its ballots
  constexpr int PF = 8;
  for (int64_t base = beg; base < end; base += PF * kWave) {
    int id[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int64_t i = base + j * kWave + lane;
      id[j] = i < end ? load_id(ids, dtype, i) : -1;
    }
#pragma unroll
    for (int j = 0; j < PF; ++j)
      if (base + j * kWave < end) place(base + j * kWave + lane, id[j]);
  }
}

// What big_plan_kernel (grouped_gemm.hip) derives from the aligned ids, derived from the
// per-expert counts instead, for an alignment with blocks of 256 slots: the m-block
// ranges [bounds[x], bounds[x+1]) of the 8 XCDs with equal estimated work (a block costs
// 38 / 48 / 64 / 64 with at most 32 / at most 64 / fewer than 256 / 256 real slots), no range
// longer than cap_mb, and the per-block counters and the status word of the one-launch form
// cleared.  Saves the
// large-tile path a launch.  Called by all kScanThreads threads; contains barriers.
constexpr int kPlanBlock = 256, kPlanXcds = 8;
__device__ void plan_from_counts(const volatile int* cum, const volatile int* tot, int E, int cap_mb,
                                 int32_t* bounds, int32_t* done, int num_done, volatile int* wave_tot) {
  __shared__ int s_b[kPlanXcds + 1];
  for (int i = threadIdx.x; i < num_done; i += kScanThreads) done[i] = 0;
  if (threadIdx.x == 0) bounds[kMoeStatusWord] = 0;  // expired waits of the one-launch form
  const int live_mb = cum[E] / kPlanBlock;
  int w = 0, nb = 0, first = 0;
  if (static_cast<int>(threadIdx.x) < E) {
    nb = (cum[threadIdx.x + 1] - cum[threadIdx.x]) / kPlanBlock;
    first = cum[threadIdx.x] / kPlanBlock;
    if (nb > 0) {
      const int r = tot[threadIdx.x] - (nb - 1) * kPlanBlock;  // real slots of the expert's last block
      w = (nb - 1) * 64 + (r <= 32 ? 38 : (r <= 64 ? 48 : 64));
    }
  }
  const int excl = block_exclusive_scan(w, wave_tot);
  const int total = wave_tot[kScanWaves];
  if (threadIdx.x <= kPlanXcds) s_b[threadIdx.x] = threadIdx.x == 0 ? 0 : live_mb;
  __syncthreads();
  if (w > 0) {
    // the block whose cost takes the running sum across x / 8 of the total is the last of XCD x - 1
#pragma unroll
    for (int x = 1; x < kPlanXcds; ++x) {
      const int64_t target = (static_cast<int64_t>(total) * x + kPlanXcds - 1) / kPlanXcds;
      if (excl < target && excl + w >= target) {
        const int j = static_cast<int>((target - excl + 63) / 64);  // full blocks cost 64 each
        s_b[x] = first + (j < nb ? j : nb);
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int x = 1; x <= kPlanXcds; ++x) s_b[x] = max(s_b[x], s_b[x - 1]);
    for (int x = 1; x <= kPlanXcds; ++x) s_b[x] = min(s_b[x], s_b[x - 1] + cap_mb);
    s_b[kPlanXcds] = live_mb;
    for (int x = kPlanXcds - 1; x >= 1; --x) s_b[x] = max(s_b[x], s_b[x + 1] - cap_mb);
    for (int x = 0; x <= kPlanXcds; ++x) bounds[x] = s_b[x];
  }
}

// The single-workgroup alignment: histogram, scans and scatter in LDS (`lds`: kScanWaves * E +
// 2 E + kScanWaves + 2 ints).  Called by all kScanThreads threads; contains barriers.
__device__ void align_small_body(const void* __restrict__ ids, int dtype, int numel, int E, int BM, int id_bits,
                                 int32_t* __restrict__ sorted_ids, int64_t sorted_cap,
                                 int32_t* __restrict__ expert_ids, int64_t expert_cap,
                                 int32_t* __restrict__ num_post_pad, int32_t* plan_bounds, int32_t* plan_done,
                                 int plan_num_done, int plan_cap_mb, int* lds) {
  // layout: seg_cnt[kScanWaves][E] | cum[E+1] | tot[E] | wave_tot[kScanWaves+1]
  volatile int* seg_cnt = lds;
  volatile int* cum = lds + kScanWaves * E;
  volatile int* tot = cum + (E + 1);
  volatile int* wave_tot = tot + E;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int seg_len = ((numel + kScanWaves - 1) / kScanWaves + kWave - 1) / kWave * kWave;
  const int beg = min(wave * seg_len, numel), end = min(beg + seg_len, numel);

  for (int i = threadIdx.x; i < kScanWaves * E; i += kScanThreads) seg_cnt[i] = 0;
  __syncthreads();
  for (int i = beg + lane; i < end; i += kWave) {
    const int id = load_id(ids, dtype, i);
    if (id >= 0 && id < E) atomicAdd(const_cast<int*>(&seg_cnt[wave * E + id]), 1);
  }
  __syncthreads();
  int padded = 0;
  if (threadIdx.x < E) {
    const int e = threadIdx.x;
    int running = 0;
    for (int w = 0; w < kScanWaves; ++w) {
      const int c = seg_cnt[w * E + e];
      seg_cnt[w * E + e] = running;
      running += c;
    }
    tot[e] = running;
    padded = (running + BM - 1) / BM * BM;
  }
  const int excl = block_exclusive_scan(padded, wave_tot);
  if (threadIdx.x < E) cum[threadIdx.x] = excl;
  if (threadIdx.x == E) cum[E] = excl;  // E < kScanThreads: threads past E add 0
  if (E == kScanThreads && threadIdx.x == 0) cum[E] = wave_tot[kScanWaves];
  __syncthreads();
  write_blocks_and_padding(cum, tot, E, BM, numel, sorted_ids, sorted_cap, expert_ids, expert_cap,
                           num_post_pad);
  if (plan_bounds) plan_from_counts(cum, tot, E, plan_cap_mb, plan_bounds, plan_done, plan_num_done, wave_tot);
  // per-wavefront running slots: segment prefix + expert base
  for (int e = lane; e < E; e += kWave) seg_cnt[wave * E + e] += cum[e];
  scatter_segment(ids, dtype, beg, end, E, id_bits, seg_cnt + wave * E, sorted_ids);
}

__global__ __launch_bounds__(kScanThreads) void align_small_kernel(
    const void* __restrict__ ids, int dtype, int numel, int E, int BM, int id_bits,
    int32_t* __restrict__ sorted_ids, int64_t sorted_cap, int32_t* __restrict__ expert_ids,
    int64_t expert_cap, int32_t* __restrict__ num_post_pad, int32_t* plan_bounds, int32_t* plan_done,
    int plan_num_done, int plan_cap_mb) {
  extern __shared__ int lds[];
  align_small_body(ids, dtype, numel, E, BM, id_bits, sorted_ids, sorted_cap, expert_ids, expert_cap, num_post_pad,
                   plan_bounds, plan_done, plan_num_done, plan_cap_mb, lds);
}

// Routing and alignment of a very small batch in one launch (such a call is a handful of short
// kernels: every launch saved is several per cent of it).  The one workgroup first routes all T
// rows, 16 wavefronts side by side with the lane layout, reduction order and results of
// topk_softmax_pow2_kernel (csrc/moe_topk_softmax_kernels.cu:182-380 of the reference); the ids
// it has written are then aligned by the same code as align_small_kernel (stores of a workgroup
// are visible to its own later loads behind a workgroup barrier).
template <int E>
__global__ __launch_bounds__(kScanThreads) void route_align_small_kernel(
    const float* __restrict__ gating, float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
    int32_t* __restrict__ tok_exp_idx, int T, int K, int renormalize, int BM, int id_bits,
    int32_t* __restrict__ sorted_ids, int64_t sorted_cap, int32_t* __restrict__ expert_ids,
    int64_t expert_cap, int32_t* __restrict__ num_post_pad, int32_t* plan_bounds, int32_t* plan_done,
    int plan_num_done, int plan_cap_mb) {
  extern __shared__ int lds[];
  using G = Pow2Geom<E>;
  constexpr int VPT = G::kVpt, TPR = G::kTpr, RPW = G::kRowsPerWave;
  constexpr int kRowsPerPass = kScanWaves * RPW;   // rows the workgroup routes side by side
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int t = lane % TPR;
  const int passes = (T + kRowsPerPass - 1) / kRowsPerPass;
  // two passes in flight: the loads of pass i + 1 are issued before pass i is routed
  float v[2][VPT];
  auto row_of = [&](int pass) { return (pass * kScanWaves + wave) * RPW + lane / TPR; };
  {
    const int r = row_of(0);
    load_row<E>(gating, r < T ? r : T - 1, t, v[0]);
  }
  for (int pass = 0; pass < passes; pass += 2) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int cur = pass + h;
      if (cur < passes) {  // the same for every thread: whole wavefronts take part in the row's exchanges
        if (cur + 1 < passes) {
          const int rn = row_of(cur + 1);
          load_row<E>(gating, rn < T ? rn : T - 1, t, v[h ^ 1]);
        }
        const int r = row_of(cur);
        route_row<E>(v[h], t, r, r < T, topk_w, topk_ids, tok_exp_idx, T, K, renormalize);
      }
    }
  }
  __syncthreads();
  align_small_body(topk_ids, MOE_ID_I32, T * K, E, BM, id_bits, sorted_ids, sorted_cap, expert_ids, expert_cap,
                   num_post_pad, plan_bounds, plan_done, plan_num_done, plan_cap_mb, lds);
}

// ---- large path -----------------------------------------------------------
__global__ __launch_bounds__(kWave) void align_count_kernel(const void* __restrict__ ids, int dtype,
                                                            int64_t numel, int E,
                                                            int32_t* __restrict__ seg_cnt) {
  extern __shared__ int lds[];
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += kWave) lds[e] = 0;
  __syncthreads();
  const int64_t beg = static_cast<int64_t>(blockIdx.x) * kSegLen;
  const int64_t end = beg + kSegLen < numel ? beg + kSegLen : numel;
  int id[kSegLen / kWave];  // all loads of the segment in flight together
#pragma unroll
  for (int j = 0; j < kSegLen / kWave; ++j) {
    const int64_t i = beg + j * kWave + lane;
    id[j] = i < end ? load_id(ids, dtype, i) : -1;
  }
#pragma unroll
  for (int j = 0; j < kSegLen / kWave; ++j)
    if (id[j] >= 0 && id[j] < E) atomicAdd(&lds[id[j]], 1);
  __syncthreads();
  for (int e = lane; e < E; e += kWave) seg_cnt[static_cast<size_t>(blockIdx.x) * E + e] = lds[e];
}

__global__ __launch_bounds__(kScanThreads) void align_scan_kernel(
    int32_t* __restrict__ seg_cnt, int nseg, int E, int BM, int numel,
    int32_t* __restrict__ cum_out, int32_t* __restrict__ sorted_ids, int64_t sorted_cap,
    int32_t* __restrict__ expert_ids, int64_t expert_cap, int32_t* __restrict__ num_post_pad) {
  __shared__ int s_cum[kMaxExperts + 1];
  __shared__ int s_tot[kMaxExperts];
  __shared__ int s_wave_tot[kScanWaves + 1];
  // per expert: exclusive prefix of its counts over segments (in place).
  // Thread t works on expert t % E and on the (t / E)-th range of segments, so
  // that a wavefront reads 64 consecutive experts of one segment (one 256-byte
  // line; indexing the lanes by segment would touch 64 lines per load).
  __shared__ int s_part[kScanThreads];
  const int R = kScanThreads / E;                 // segment ranges (E <= kScanThreads)
  const int L = (nseg + R - 1) / R;               // segments per range
  const int e = threadIdx.x % E, r = threadIdx.x / E;
  const bool active = r < R;
  const int sbeg = r * L, send = min(nseg, sbeg + L);
  // counts are fetched eight at a time: issued one by one, each load would wait for the one before
  constexpr int CH = 8;
  int sum = 0;
  if (active) {
    for (int sg0 = sbeg; sg0 < send; sg0 += CH) {
      int c[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) c[i] = sg0 + i < send ? seg_cnt[static_cast<size_t>(sg0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < CH; ++i) sum += c[i];
    }
    s_part[r * E + e] = sum;
  }
  __syncthreads();
  if (active) {
    int running = 0, total = 0;
    for (int q = 0; q < R; ++q) {
      const int v = s_part[q * E + e];
      if (q < r) running += v;
      total += v;
    }
    if (r == 0) s_tot[e] = total;
    for (int sg0 = sbeg; sg0 < send; sg0 += CH) {
      int c[CH];
#pragma unroll
      for (int i = 0; i < CH; ++i) c[i] = sg0 + i < send ? seg_cnt[static_cast<size_t>(sg0 + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        if (sg0 + i < send) seg_cnt[static_cast<size_t>(sg0 + i) * E + e] = running;
        running += c[i];
      }
    }
  }
  __syncthreads();
  int padded = 0;
  if (threadIdx.x < E) padded = (s_tot[threadIdx.x] + BM - 1) / BM * BM;
  const int excl = block_exclusive_scan(padded, s_wave_tot);
  if (threadIdx.x < E) s_cum[threadIdx.x] = excl;
  if (threadIdx.x == E) s_cum[E] = excl;
  if (E == kScanThreads && threadIdx.x == 0) s_cum[E] = s_wave_tot[kScanWaves];
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += kScanThreads) cum_out[e] = s_cum[e];
  write_blocks_and_padding(s_cum, s_tot, E, BM, numel, sorted_ids, sorted_cap, expert_ids,
                           expert_cap, num_post_pad);
}

// Scan and scatter in one launch: every workgroup owns kScanWaves consecutive
// segments and derives what it needs from the per-segment histograms by itself
// (they are a few tens of KB and sit in L2): the totals per expert, the counts
// in front of its own segments, the padded prefix over experts.  Then each of
// its wavefronts scatters one segment, and the workgroups share the padding and
// expert_ids writes.  No workgroup waits for another.
// LDS: part[nwg][E] | own[kScanWaves][E] | cum[E+1] | tot[E] | wave_tot[kScanWaves+1]
__global__ __launch_bounds__(kScanThreads) void align_place_kernel(
    const void* __restrict__ ids, int dtype, int64_t numel, int E, int BM, int id_bits,
    const int32_t* __restrict__ seg_cnt, int nseg, int32_t* __restrict__ sorted_ids,
    int64_t sorted_cap, int32_t* __restrict__ expert_ids, int64_t expert_cap,
    int32_t* __restrict__ num_post_pad, int32_t* plan_bounds, int32_t* plan_done, int plan_num_done,
    int plan_cap_mb) {
  extern __shared__ int lds[];
  const int nwg = gridDim.x;
  volatile int* part = lds;
  volatile int* own = lds + nwg * E;
  volatile int* cum = own + kScanWaves * E;
  volatile int* tot = cum + (E + 1);
  volatile int* wave_tot = tot + E;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  // thread t sums expert t % E over the segments of workgroups t / E, t / E + R, ...
  // (a wavefront reads 64 consecutive experts of one segment: one 256-byte line)
  const int R = kScanThreads / E;
  const int e = threadIdx.x % E, r = threadIdx.x / E;
  if (r < R) {
    for (int q = r; q < nwg; q += R) {
      const int s0 = q * kScanWaves;
      int c[kScanWaves];
#pragma unroll
      for (int i = 0; i < kScanWaves; ++i)
        c[i] = s0 + i < nseg ? seg_cnt[static_cast<size_t>(s0 + i) * E + e] : 0;
      int sum = 0;
#pragma unroll
      for (int i = 0; i < kScanWaves; ++i) sum += c[i];
      part[q * E + e] = sum;
      if (q == static_cast<int>(blockIdx.x)) {
#pragma unroll
        for (int i = 0; i < kScanWaves; ++i) own[i * E + e] = c[i];
      }
    }
  }
  __syncthreads();
  int padded = 0;
  if (threadIdx.x < E) {
    int before = 0, total = 0;
    for (int q = 0; q < nwg; ++q) {
      const int v = part[q * E + threadIdx.x];
      if (q < static_cast<int>(blockIdx.x)) before += v;
      total += v;
    }
    tot[threadIdx.x] = total;
    padded = (total + BM - 1) / BM * BM;
    // own[w][e] becomes the number of ids of expert e in front of segment w of this workgroup
    int running = before;
    for (int w = 0; w < kScanWaves; ++w) {
      const int c = own[w * E + threadIdx.x];
      own[w * E + threadIdx.x] = running;
      running += c;
    }
  }
  const int excl = block_exclusive_scan(padded, wave_tot);
  if (threadIdx.x < E) cum[threadIdx.x] = excl;
  if (threadIdx.x == E) cum[E] = excl;  // E < kScanThreads: threads past E add 0
  if (E == kScanThreads && threadIdx.x == 0) cum[E] = wave_tot[kScanWaves];
  __syncthreads();
  // this workgroup's share of expert_ids, of the padding inside the experts' last
  // blocks and of the tail behind the padded total
  const int total = cum[E];
  if (blockIdx.x == 0 && threadIdx.x == 0) *num_post_pad = total;
  const int used_blocks = total / BM;
  const int64_t gtid = static_cast<int64_t>(blockIdx.x) * kScanThreads + threadIdx.x;
  const int64_t gthreads = static_cast<int64_t>(nwg) * kScanThreads;
  for (int64_t b = gtid; b < expert_cap; b += gthreads) {
    int owner = 0;
    if (b < used_blocks) {
      const int pos = static_cast<int>(b) * BM;
      int lo = 1, hi = E;  // first j in [1, E] with cum[j] > pos; the block belongs to expert j - 1
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (cum[mid] > pos) hi = mid; else lo = mid + 1;
      }
      owner = lo - 1;
    }
    expert_ids[b] = owner;
  }
  for (int x = blockIdx.x * kScanWaves + wave; x < E; x += nwg * kScanWaves) {
    const int beg = cum[x] + tot[x], end = cum[x + 1];
    for (int p = beg + lane; p < end; p += kWave) sorted_ids[p] = static_cast<int32_t>(numel);
  }
  for (int64_t p = total + gtid; p < sorted_cap; p += gthreads) sorted_ids[p] = static_cast<int32_t>(numel);
  if (plan_bounds && blockIdx.x == 0)
    plan_from_counts(cum, tot, E, plan_cap_mb, plan_bounds, plan_done, plan_num_done, wave_tot);
  // per-wavefront running slots: ids in front of the segment + expert base
  const int sg = blockIdx.x * kScanWaves + wave;
  if (sg >= nseg) return;
  for (int x = lane; x < E; x += kWave) own[wave * E + x] += cum[x];
  const int64_t beg = static_cast<int64_t>(sg) * kSegLen;
  const int64_t end = beg + kSegLen < numel ? beg + kSegLen : numel;
  scatter_segment(ids, dtype, beg, end, E, id_bits, own + wave * E, sorted_ids);
}

__global__ __launch_bounds__(kWave) void align_scatter_kernel(
    const void* __restrict__ ids, int dtype, int64_t numel, int E, int id_bits,
    const int32_t* __restrict__ seg_base, const int32_t* __restrict__ cum,
    int32_t* __restrict__ sorted_ids) {
  extern __shared__ int lds[];
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += kWave)
    lds[e] = seg_base[static_cast<size_t>(blockIdx.x) * E + e] + cum[e];
  __syncthreads();
  const int64_t beg = static_cast<int64_t>(blockIdx.x) * kSegLen;
  const int64_t end = beg + kSegLen < numel ? beg + kSegLen : numel;
  scatter_segment(ids, dtype, beg, end, E, id_bits, lds, sorted_ids);
}

int bits_for(int E) {
  int b = 1;
  while ((1 << b) < E) ++b;
  return b;
}

}  // namespace

MOE_EXPORT int64_t moe_align_workspace_bytes(int64_t numel, int E) {
  if (numel < 0 || E < 1) return 0;
  if (numel <= kSmallNumel && E <= kSmallMaxExperts) return 0;
  const int64_t nseg = numel > 0 ? (numel + kSegLen - 1) / kSegLen : 1;
  return moe_align_up((nseg * E + E + 1) * static_cast<int64_t>(sizeof(int32_t)), 256);
}

static int align_impl(const void* topk_ids, int ids_dtype, int64_t numel, int E, int block_size,
                      int32_t* sorted_token_ids, int64_t sorted_cap, int32_t* expert_ids,
                      int64_t expert_cap, int32_t* num_tokens_post_pad, void* workspace,
                      int64_t workspace_bytes, void* stream, int32_t* plan_bounds, int32_t* plan_done,
                      int plan_num_done, int plan_cap_mb) {
  if (numel < 0 || E < 1 || block_size < 1)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: bad sizes numel=%lld E=%d block_size=%d",
                    static_cast<long long>(numel), E, block_size);
  if (E > kMaxExperts)
    return moe_fail(MOE_ERR_UNSUPPORTED, "moe_align_block_size: num_experts %d > %d", E, kMaxExperts);
  if (ids_dtype < MOE_ID_I32 || ids_dtype > MOE_ID_U8)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: unknown id dtype code %d", ids_dtype);
  const int64_t need_sorted = numel + static_cast<int64_t>(E) * (block_size - 1);
  if (need_sorted > INT32_MAX)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: padded length overflows int32");
  if (sorted_cap < need_sorted)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: sorted_token_ids holds %lld, needs %lld",
                    static_cast<long long>(sorted_cap), static_cast<long long>(need_sorted));
  if (expert_cap < (need_sorted + block_size - 1) / block_size)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: expert_ids holds %lld, needs %lld",
                    static_cast<long long>(expert_cap),
                    static_cast<long long>((need_sorted + block_size - 1) / block_size));
  // (an empty output - no ids and blocks of one slot - may come with a null pointer)
  if ((need_sorted > 0 && (!sorted_token_ids || !expert_ids)) || !num_tokens_post_pad || (numel > 0 && !topk_ids))
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int id_bits = bits_for(E);
  if (numel <= kSmallNumel && E <= kSmallMaxExperts) {
    const size_t lds = (static_cast<size_t>(kScanWaves) * E + (E + 1) + E + kScanWaves + 1) * sizeof(int);
    hipLaunchKernelGGL(align_small_kernel, dim3(1), dim3(kScanThreads), lds, s, topk_ids, ids_dtype,
                       static_cast<int>(numel), E, block_size, id_bits, sorted_token_ids,
                       sorted_cap, expert_ids, expert_cap, num_tokens_post_pad, plan_bounds, plan_done,
                       plan_num_done, plan_cap_mb);
    return moe_check_launch("moe_align_block_size (single workgroup)");
  }
  const int64_t need_ws = moe_align_workspace_bytes(numel, E);
  if (!workspace || workspace_bytes < need_ws)
    return moe_fail(MOE_ERR_WORKSPACE, "moe_align_block_size: workspace %lld B, needs %lld B",
                    static_cast<long long>(workspace_bytes), static_cast<long long>(need_ws));
  const int nseg = numel > 0 ? static_cast<int>((numel + kSegLen - 1) / kSegLen) : 1;
  int32_t* seg_cnt = static_cast<int32_t*>(workspace);
  int32_t* cum = seg_cnt + static_cast<size_t>(nseg) * E;
  hipLaunchKernelGGL(align_count_kernel, dim3(nseg), dim3(kWave), E * sizeof(int), s, topk_ids,
                     ids_dtype, numel, E, seg_cnt);
  // scan and scatter as one launch while its LDS tables fit
  const int nwg = (nseg + kScanWaves - 1) / kScanWaves;
  const size_t place_lds = (static_cast<size_t>(nwg + kScanWaves) * E + (E + 1) + E + kScanWaves + 1) * sizeof(int);
  if (place_lds <= 60 * 1024) {
    hipLaunchKernelGGL(align_place_kernel, dim3(nwg), dim3(kScanThreads), place_lds, s, topk_ids, ids_dtype,
                       numel, E, block_size, id_bits, seg_cnt, nseg, sorted_token_ids, sorted_cap,
                       expert_ids, expert_cap, num_tokens_post_pad, plan_bounds, plan_done, plan_num_done,
                       plan_cap_mb);
    return moe_check_launch("moe_align_block_size (count + place)");
  }
  hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, seg_cnt, nseg, E,
                     block_size, static_cast<int>(numel), cum, sorted_token_ids, sorted_cap,
                     expert_ids, expert_cap, num_tokens_post_pad);
  hipLaunchKernelGGL(align_scatter_kernel, dim3(nseg), dim3(kWave), E * sizeof(int), s, topk_ids,
                     ids_dtype, numel, E, id_bits, seg_cnt, cum,
                     sorted_token_ids);
  return moe_check_launch("moe_align_block_size");
}

MOE_EXPORT int moe_align_block_size(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                                    int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                    int32_t* expert_ids, int64_t expert_cap,
                                    int32_t* num_tokens_post_pad, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
  return align_impl(topk_ids, ids_dtype, numel, E, block_size, sorted_token_ids, sorted_cap, expert_ids,
                    expert_cap, num_tokens_post_pad, workspace, workspace_bytes, stream, nullptr, nullptr, 0, 0);
}

// Whether moe_align_block_size_planned can serve this size (its kernels keep per-expert
// tables in LDS); otherwise align without a plan.
MOE_EXPORT int moe_align_can_plan(int64_t numel, int E) {
  if (numel < 0 || E < 1 || E > kMaxExperts) return 0;
  if (numel <= kSmallNumel && E <= kSmallMaxExperts) return 1;
  const int64_t nseg = numel > 0 ? (numel + kSegLen - 1) / kSegLen : 1;
  const int64_t nwg = (nseg + kScanWaves - 1) / kScanWaves;
  return (static_cast<size_t>(nwg + kScanWaves) * E + (E + 1) + E + kScanWaves + 1) * sizeof(int) <= 60 * 1024;
}

MOE_EXPORT int moe_align_block_size_planned(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                                            int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                            int32_t* expert_ids, int64_t expert_cap,
                                            int32_t* num_tokens_post_pad, void* workspace,
                                            int64_t workspace_bytes, void* stream, int32_t* plan_bounds,
                                            int32_t* plan_done, int plan_num_done, int plan_cap_mb) {
  if (block_size != kPlanBlock || !plan_bounds || !plan_done || plan_num_done < 0 || plan_cap_mb < 1)
    return moe_fail(MOE_ERR_ARG, "moe_align_block_size_planned: needs block_size %d and the plan buffers",
                    kPlanBlock);
  if (!moe_align_can_plan(numel, E))
    return moe_fail(MOE_ERR_UNSUPPORTED, "moe_align_block_size_planned: %d experts x %lld ids is beyond the "
                    "kernels that can plan; align without a plan", E, static_cast<long long>(numel));
  return align_impl(topk_ids, ids_dtype, numel, E, block_size, sorted_token_ids, sorted_cap, expert_ids,
                    expert_cap, num_tokens_post_pad, workspace, workspace_bytes, stream, plan_bounds,
                    plan_done, plan_num_done, plan_cap_mb);
}

// Routing (moe_topk_softmax) and alignment (moe_align_block_size, with the plan of
// moe_align_block_size_planned when plan_bounds is given) of a small batch as one launch.
MOE_EXPORT int moe_route_align_supported(int T, int E, int K) {
  if (T < 1 || T > kRouteAlignMaxTokens || E < 1 || E > 256 || (E & (E - 1)) != 0 || K < 1 || K > E) return 0;
  return static_cast<int64_t>(T) * K <= kSmallNumel ? 1 : 0;
}

template <int E>
static void launch_route_align(const float* g, float* w, int32_t* ids, int32_t* tei, int T, int K, int renorm, int BM,
                               int32_t* sorted, int64_t sorted_cap, int32_t* eids, int64_t expert_cap, int32_t* npp,
                               int32_t* pb, int32_t* pd, int pnd, int pcap, hipStream_t s) {
  const size_t lds = (static_cast<size_t>(kScanWaves) * E + (E + 1) + E + kScanWaves + 1) * sizeof(int);
  hipLaunchKernelGGL(route_align_small_kernel<E>, dim3(1), dim3(kScanThreads), lds, s, g, w, ids, tei, T, K, renorm, BM,
                     bits_for(E), sorted, sorted_cap, eids, expert_cap, npp, pb, pd, pnd, pcap);
}

MOE_EXPORT int moe_route_align_block_size(const float* gating_output, float* topk_weights, int32_t* topk_ids,
                                          int32_t* token_expert_indices, int T, int E, int K, int renormalize,
                                          int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                          int32_t* expert_ids, int64_t expert_cap, int32_t* num_tokens_post_pad,
                                          void* stream, int32_t* plan_bounds, int32_t* plan_done, int plan_num_done,
                                          int plan_cap_mb) {
  if (!moe_route_align_supported(T, E, K))
    return moe_fail(MOE_ERR_UNSUPPORTED, "route_align_block_size: T=%d E=%d K=%d (at most %d tokens, a power-of-two "
                    "number of experts up to 256, T*K <= %lld); route and align apart", T, E, K, kRouteAlignMaxTokens,
                    static_cast<long long>(kSmallNumel));
  if (block_size < 1) return moe_fail(MOE_ERR_ARG, "route_align_block_size: block_size %d", block_size);
  if (!gating_output || !topk_weights || !topk_ids || !token_expert_indices || !sorted_token_ids || !expert_ids ||
      !num_tokens_post_pad)
    return moe_fail(MOE_ERR_ARG, "route_align_block_size: null pointer");
  if (plan_bounds && (block_size != kPlanBlock || !plan_done || plan_num_done < 0 || plan_cap_mb < 1))
    return moe_fail(MOE_ERR_ARG, "route_align_block_size: a plan needs block_size %d and the plan buffers", kPlanBlock);
  const int64_t need_sorted = static_cast<int64_t>(T) * K + static_cast<int64_t>(E) * (block_size - 1);
  if (need_sorted > INT32_MAX) return moe_fail(MOE_ERR_ARG, "route_align_block_size: padded length overflows int32");
  if (sorted_cap < need_sorted || expert_cap < (need_sorted + block_size - 1) / block_size)
    return moe_fail(MOE_ERR_ARG, "route_align_block_size: sorted_token_ids holds %lld (needs %lld), expert_ids %lld "
                    "(needs %lld)", static_cast<long long>(sorted_cap), static_cast<long long>(need_sorted),
                    static_cast<long long>(expert_cap), static_cast<long long>((need_sorted + block_size - 1) / block_size));
  hipStream_t s = static_cast<hipStream_t>(stream);
#define MOE_ROUTE_ALIGN_CASE(N)                                                                                        \
  case N:                                                                                                              \
    launch_route_align<N>(gating_output, topk_weights, topk_ids, token_expert_indices, T, K, renormalize, block_size,  \
                          sorted_token_ids, sorted_cap, expert_ids, expert_cap, num_tokens_post_pad, plan_bounds,      \
                          plan_done, plan_num_done, plan_cap_mb, s);                                                   \
    break;
  switch (E) {
    MOE_ROUTE_ALIGN_CASE(1) MOE_ROUTE_ALIGN_CASE(2) MOE_ROUTE_ALIGN_CASE(4) MOE_ROUTE_ALIGN_CASE(8)
    MOE_ROUTE_ALIGN_CASE(16) MOE_ROUTE_ALIGN_CASE(32) MOE_ROUTE_ALIGN_CASE(64) MOE_ROUTE_ALIGN_CASE(128)
    MOE_ROUTE_ALIGN_CASE(256)
    default: return moe_fail(MOE_ERR_UNSUPPORTED, "route_align_block_size: E=%d", E);
  }
#undef MOE_ROUTE_ALIGN_CASE
  return moe_check_launch("route_align_block_size");
}

// ---------------------------------------------------------------------------
// Allocation-free variant: the per-segment histograms of the large path live in a
// file-scope device array instead of a caller-provided workspace.  Each GPU the
// library runs on holds its own copy of the array (at its own address) until the
// process ends.
// ---------------------------------------------------------------------------
constexpr int64_t kStaticScratchBytes = 4 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// device address of `scratch` per device; the array's name is only a host-side handle
static std::atomic<void*> g_scratch_ptr[kMoeMaxDevices];

static int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return moe_fail(MOE_ERR_LAUNCH, "moe_align_block_size_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMoeMaxDevices)
    return moe_fail(MOE_ERR_UNSUPPORTED, "moe_align_block_size_static: device %d beyond the %d this entry point tracks", dev, kMoeMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    // once per device, with that device current
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return moe_fail(MOE_ERR_LAUNCH, "moe_align_block_size_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // two threads storing the same address is harmless
  }
  *out = p;
  return MOE_OK;
}

MOE_EXPORT int moe_align_block_size_static(const void* topk_ids, int ids_dtype, int64_t numel, int E,
                                           int block_size, int32_t* sorted_token_ids, int64_t sorted_cap,
                                           int32_t* expert_ids, int64_t expert_cap,
                                           int32_t* num_tokens_post_pad, void* stream) {
  const int64_t need = moe_align_workspace_bytes(numel, E);
  if (need > kStaticScratchBytes)
    return moe_fail(MOE_ERR_WORKSPACE, "moe_align_block_size_static: %lld ids over %d experts need %lld B of scratch, "
                    "the built-in buffer holds %lld B; use moe_align_block_size with a workspace",
                    static_cast<long long>(numel), E, static_cast<long long>(need),
                    static_cast<long long>(kStaticScratchBytes));
  void* ws = nullptr;
  if (need > 0) {
    if (int rc = static_scratch(&ws)) return rc;
  }
  // the count kernel writes every histogram entry the later kernels read: nothing has to start at zero
  return align_impl(topk_ids, ids_dtype, numel, E, block_size, sorted_token_ids, sorted_cap, expert_ids,
                    expert_cap, num_tokens_post_pad, ws, need, stream, nullptr, nullptr, 0, 0);
}
