// Expert sort (moe_align_block_size): stable counting sort of the flat slot
// indices by expert, every expert segment padded to a multiple of block_size.
//
// One workgroup of 16 wavefronts.  Wave w owns the contiguous chunk
// [w*chunk, (w+1)*chunk) of topk_ids:
//   pass 1  per-wave histogram with ballots           -> LDS hist[wave][expert]
//   scan    exclusive prefix over waves per expert, padded exclusive prefix
//           over experts                               -> LDS base[wave][expert]
//   pass 2  each wave re-walks its chunk; lane e keeps the running write
//           position of expert e, a slot's position is that value (read with a
//           lane shuffle) plus its rank among equal experts in the 64-wide step.
// Chunks are contiguous and walked in ascending order, so the sort is stable,
// as the reference's per-thread chunks are (src/moe_align_block_size.hip:78-135).
// Output conventions follow the reference wrapper
// (layers/moe/moe_align_block_size.py:32-48): pads and tail of sorted ids are -1,
// unused tail of expert_ids is 0.
#include "common.h"
#include "router_device.h"

namespace em {
namespace {

constexpr int kAlignThreads = 1024;
constexpr int kAlignWaves = kAlignThreads / kWave;

// The sort, run by one workgroup of kAlignThreads threads; `ids` may live in global memory or in LDS.
// hist: pass 1 counts, then write bases; seg_begin: padded exclusive prefix (both in LDS).
// EC: the number of experts as a compile-time constant (the ballot loops unroll), 0 = use the argument
template <typename IdT, int EC>
__device__ __forceinline__ void align_body(
    const IdT* __restrict__ ids, int64_t numel, int E_arg, int block,
    int32_t* __restrict__ sorted, int64_t sorted_len, int32_t* __restrict__ expert_ids,
    int64_t eid_len, int32_t* __restrict__ post_pad, int32_t* __restrict__ seg_out,
    int32_t (*hist)[kMaxExperts], int32_t* seg_begin) {

    const int E = EC ? EC : E_arg;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));

    const int64_t chunk = round_up(ceil_div(numel, kAlignWaves), kWave);
    const int64_t begin = wave * chunk;
    const int64_t end = (begin + chunk < numel) ? begin + chunk : numel;

    // every output element is defined by this kernel: start from the pad values
    for (int64_t i = tid; i < sorted_len; i += kAlignThreads) sorted[i] = -1;
    for (int64_t i = tid; i < eid_len; i += kAlignThreads) expert_ids[i] = 0;

    // ---- pass 1: per-wave histogram (lane e accumulates expert e) ----
    int32_t cnt = 0;
    for (int64_t i0 = begin; i0 < end; i0 += kWave) {
        const int64_t i = i0 + lane;
        const int e = (i < end) ? static_cast<int>(ids[i]) : -1;
        auto count_expert = [&](int j) {
            const uint64_t m = __ballot(e == j);
            if (lane == j) cnt += __popcll(m);
        };
        if (EC) {
#pragma unroll
            for (int j = 0; j < EC; ++j) count_expert(j);
        } else {
            for (int j = 0; j < E; ++j) count_expert(j);
        }
    }
    if (lane < kMaxExperts) hist[wave][lane] = (lane < E) ? cnt : 0;
    __syncthreads();

    // ---- scan: thread e turns counts into per-wave write bases ----
    int32_t total = 0;
    if (tid < E) {
        for (int w = 0; w < kAlignWaves; ++w) {
            const int32_t c = hist[w][tid];
            hist[w][tid] = total;  // exclusive prefix over waves
            total += c;
        }
        seg_begin[tid + 1] = static_cast<int32_t>(round_up(total, block));
    }
    if (tid == 0) seg_begin[0] = 0;
    __syncthreads();
    if (tid == 0) {
        int32_t run = 0;
        for (int e = 0; e < E; ++e) {
            const int32_t padded = seg_begin[e + 1];
            seg_begin[e] = run;
            run += padded;
        }
        seg_begin[E] = run;
        post_pad[0] = run;
    }
    __syncthreads();  // also orders the -1 / 0 fill before the scatter below
    if (seg_out != nullptr && tid <= E) seg_out[tid] = seg_begin[tid];  // padded start of every expert segment

    // block -> expert table: every thread looks its blocks up in the segment starts (a hot expert has
    // thousands of blocks: one thread per expert would walk them alone)
    {
        const int64_t nblocks = seg_begin[E] / block;
        for (int64_t b = tid; b < nblocks && b < eid_len; b += kAlignThreads) {
            const int32_t row = static_cast<int32_t>(b) * block;
            int e = 0;
            while (e + 1 < E && row >= seg_begin[e + 1]) ++e;
            expert_ids[b] = e;
        }
    }

    // ---- pass 2: stable scatter ----
    int32_t pos = (lane < E) ? seg_begin[lane] + hist[wave][lane] : 0;
    for (int64_t i0 = begin; i0 < end; i0 += kWave) {
        const int64_t i = i0 + lane;
        const int e = (i < end) ? static_cast<int>(ids[i]) : -1;
        const bool valid = (e >= 0 && e < E);
        const int32_t base = __shfl(pos, valid ? e : 0);
        int32_t rank = 0;
        auto rank_expert = [&](int j) {
            const uint64_t m = __ballot(e == j);
            if (e == j) rank = __popcll(m & lt_mask);
            if (lane == j) pos += __popcll(m);
        };
        if (EC) {
#pragma unroll
            for (int j = 0; j < EC; ++j) rank_expert(j);
        } else {
            for (int j = 0; j < E; ++j) rank_expert(j);
        }
        if (valid && base + rank < sorted_len) sorted[base + rank] = static_cast<int32_t>(i);
    }
}

template <typename IdT, int EC>
__global__ __launch_bounds__(kAlignThreads) void align_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E_arg, int block,
    int32_t* __restrict__ sorted, int64_t sorted_len, int32_t* __restrict__ expert_ids,
    int64_t eid_len, int32_t* __restrict__ post_pad, int32_t* __restrict__ seg_out,
    int32_t* __restrict__ counters /* the layer call's kLayerCounters counters to clear, or null */) {
    __shared__ int32_t hist[kAlignWaves][kMaxExperts];
    __shared__ int32_t seg_begin[kMaxExperts + 1];
    if (counters != nullptr && threadIdx.x < kLayerCounters) counters[threadIdx.x] = 0;
    align_body<IdT, EC>(ids, numel, E_arg, block, sorted, sorted_len, expert_ids, eid_len, post_pad, seg_out, hist,
                        seg_begin);
}

// Router and sort in one launch for batches whose k * T selected experts fit LDS (the layer then starts its
// GEMMs one kernel launch earlier: a few microseconds of a decode step).  Eight experts: eight lanes per token
// as in the stand-alone router; the selected ids go to LDS, from there to topk_ids and into the sort.
constexpr int kFusedMaxSlots = 4096;
template <typename Elem>
__global__ __launch_bounds__(kAlignThreads) void route_align_kernel(
    const typename Elem::storage* __restrict__ logits, int64_t T, int k, int renorm, float* __restrict__ out_w,
    int32_t* __restrict__ out_ids, int block, int32_t* __restrict__ sorted, int64_t sorted_len,
    int32_t* __restrict__ expert_ids, int64_t eid_len, int32_t* __restrict__ post_pad,
    int32_t* __restrict__ seg_out, int32_t* __restrict__ counters) {
    constexpr int E = 8, G = 8, kTokens = kWave / G;
    __shared__ int32_t hist[kAlignWaves][kMaxExperts];
    __shared__ int32_t seg_begin[kMaxExperts + 1];
    __shared__ int32_t ids[kFusedMaxSlots];
    const int tid = threadIdx.x;
    if (counters != nullptr && tid < kLayerCounters) counters[tid] = 0;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    for (int64_t t0 = 0; t0 < T; t0 += kAlignWaves * kTokens) {  // same trip count for every wave
        const int64_t t = t0 + wave * kTokens + lane / G;
        const bool valid = t < T;
        float v = -INFINITY;
        if (valid) {
            v = Elem::load(logits[t * E + (lane & (G - 1))]);
            if (v != v) v = -INFINITY;  // a NaN logit can never be selected
        }
        route_group<G>(v, lane, t, valid, E, k, renorm, out_w, ids);
    }
    __syncthreads();
    const int64_t numel = T * k;
    for (int64_t i = tid; i < numel; i += kAlignThreads) out_ids[i] = ids[i];
    align_body<int32_t, E>(ids, numel, E, block, sorted, sorted_len, expert_ids, eid_len, post_pad, seg_out, hist,
                           seg_begin);
}


// ---- the sort on several workgroups, for the layer call, whose workspace has room for the histogram ----
// The one-workgroup kernel above walks numel / 16 ids per wave twice (T = 8192: 19 us, T = 32768: 62 us).  Here
// a wave owns kUnitIds consecutive ids: the count kernel writes one histogram row per wave, the scatter kernel
// adds up the rows in front of a wave's own (per workgroup first, then per wave) and scatters its ids.  Waves are
// numbered in id order, so the sort is the same stable one; the two launches write the same bytes as align_kernel.
constexpr int kMwWaves = 4;                      // waves per workgroup
constexpr int kUnitIds = 256;                    // ids per wave
constexpr int kMwGroupIds = kMwWaves * kUnitIds;  // ids per workgroup

template <int EC>
__global__ __launch_bounds__(kMwWaves* kWave) void align_count_kernel(const int32_t* __restrict__ ids, int64_t numel,
                                                                      int E_arg, int32_t* __restrict__ unit_hist,
                                                                      int32_t* __restrict__ group_hist) {
    const int E = EC ? EC : E_arg;
    __shared__ int32_t wave_cnt[kMwWaves][kMaxExperts];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int64_t unit = static_cast<int64_t>(blockIdx.x) * kMwWaves + wave;
    const int64_t begin = unit * kUnitIds;
    const int64_t end = (begin + kUnitIds < numel) ? begin + kUnitIds : numel;
    int32_t cnt = 0;
    for (int64_t i0 = begin; i0 < end; i0 += kWave) {
        const int64_t i = i0 + lane;
        const int e = (i < end) ? ids[i] : -1;
        auto count_expert = [&](int j) {
            const uint64_t m = __ballot(e == j);
            if (lane == j) cnt += __popcll(m);
        };
        if (EC) {
#pragma unroll
            for (int j = 0; j < EC; ++j) count_expert(j);
        } else {
            for (int j = 0; j < E; ++j) count_expert(j);
        }
    }
    if (lane < E) {
        unit_hist[unit * E + lane] = cnt;
        wave_cnt[wave][lane] = cnt;
    }
    __syncthreads();
    if (threadIdx.x < E) {
        int32_t s = 0;
#pragma unroll
        for (int w = 0; w < kMwWaves; ++w) s += wave_cnt[w][threadIdx.x];
        group_hist[static_cast<int64_t>(blockIdx.x) * E + threadIdx.x] = s;
    }
}

template <int EC>
__global__ __launch_bounds__(kMwWaves* kWave) void align_scatter_kernel(
    const int32_t* __restrict__ ids, int64_t numel, int E_arg, int block, const int32_t* __restrict__ unit_hist,
    const int32_t* __restrict__ group_hist, int32_t* __restrict__ sorted, int64_t sorted_len,
    int32_t* __restrict__ expert_ids, int64_t eid_len, int32_t* __restrict__ post_pad, int32_t* __restrict__ seg_out,
    int32_t* __restrict__ counters) {
    const int E = EC ? EC : E_arg;
    __shared__ int32_t seg_begin[kMaxExperts + 1];  // padded start of every expert segment
    __shared__ int32_t count[kMaxExperts];          // ids of every expert in the whole batch
    __shared__ int32_t before[kMaxExperts];         // ... in the workgroups in front of this one
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int ngroups = gridDim.x;
    if (tid < E) {
        int32_t total = 0, front = 0;
        for (int g = 0; g < ngroups; ++g) {
            const int32_t c = group_hist[static_cast<int64_t>(g) * E + tid];
            if (g < static_cast<int>(blockIdx.x)) front += c;
            total += c;
        }
        count[tid] = total;
        before[tid] = front;
    }
    __syncthreads();
    if (tid == 0) {
        int32_t run = 0;
        for (int e = 0; e < E; ++e) {
            seg_begin[e] = run;
            run += static_cast<int32_t>(round_up(count[e], block));
        }
        seg_begin[E] = run;
    }
    __syncthreads();
    const int32_t total_pad = seg_begin[E];
    const int threads_all = ngroups * kMwWaves * kWave;
    const int gtid = static_cast<int>(blockIdx.x) * kMwWaves * kWave + tid;
    if (blockIdx.x == 0) {
        if (tid == 0) post_pad[0] = total_pad;
        if (seg_out != nullptr && tid <= E) seg_out[tid] = seg_begin[tid];
        if (counters != nullptr && tid < kLayerCounters) counters[tid] = 0;
        // the pad rows behind every expert's ids
        for (int e = 0; e < E; ++e)
            for (int64_t i = seg_begin[e] + count[e] + tid; i < seg_begin[e + 1] && i < sorted_len; i += kMwWaves * kWave)
                sorted[i] = -1;
    }
    // the tail of both outputs and the block -> expert table, dealt to all threads of the launch
    for (int64_t i = total_pad + gtid; i < sorted_len; i += threads_all) sorted[i] = -1;
    const int64_t nblocks = total_pad / block;
    for (int64_t b = gtid; b < eid_len; b += threads_all) {
        int e = 0;
        if (b < nblocks) {
            const int32_t row = static_cast<int32_t>(b) * block;
            while (e + 1 < E && row >= seg_begin[e + 1]) ++e;
        }
        expert_ids[b] = e;
    }
    // stable scatter of this wave's ids: lane e carries the write position of expert e
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));
    const int64_t unit0 = static_cast<int64_t>(blockIdx.x) * kMwWaves;
    int32_t pos = 0;
    if (lane < E) {
        pos = seg_begin[lane] + before[lane];
        for (int w = 0; w < wave; ++w) pos += unit_hist[(unit0 + w) * E + lane];
    }
    const int64_t begin = (unit0 + wave) * kUnitIds;
    const int64_t end = (begin + kUnitIds < numel) ? begin + kUnitIds : numel;
    for (int64_t i0 = begin; i0 < end; i0 += kWave) {
        const int64_t i = i0 + lane;
        const int e = (i < end) ? ids[i] : -1;
        const bool valid = (e >= 0 && e < E);
        const int32_t base = __shfl(pos, valid ? e : 0);
        int32_t rank = 0;
        auto rank_expert = [&](int j) {
            const uint64_t m = __ballot(e == j);
            if (e == j) rank = __popcll(m & lt_mask);
            if (lane == j) pos += __popcll(m);
        };
        if (EC) {
#pragma unroll
            for (int j = 0; j < EC; ++j) rank_expert(j);
        } else {
            for (int j = 0; j < E; ++j) rank_expert(j);
        }
        if (valid && base + rank < sorted_len) sorted[base + rank] = static_cast<int32_t>(i);
    }
}

}  // namespace

int64_t align_scratch_ints(int64_t numel, int E) {
    const int64_t groups = ceil_div(numel, kMwGroupIds);
    return groups * (kMwWaves + 1) * E;
}

int launch_align_multi(const int32_t* ids, int64_t numel, int E, int block, int32_t* sorted, int64_t sorted_len,
                       int32_t* expert_ids, int64_t eid_len, int32_t* post_pad, int32_t* seg_out, int32_t* counters,
                       int32_t* scratch, hipStream_t s) {
    const int64_t groups = ceil_div(numel, kMwGroupIds);
    if (groups < 1 || groups > 65535) return EM_ERR_UNSUPPORTED;
    int32_t* unit_hist = scratch;                                // [groups * kMwWaves][E]
    int32_t* group_hist = scratch + groups * kMwWaves * E;       // [groups][E]
    const dim3 grid(static_cast<unsigned>(groups)), blk(kMwWaves * kWave);
    if (E == 8) {
        launch(align_count_kernel<8>, grid, blk, 0, s, ids, numel, E, unit_hist, group_hist);
        launch(align_scatter_kernel<8>, grid, blk, 0, s, ids, numel, E, block, unit_hist, group_hist, sorted, sorted_len,
               expert_ids, eid_len, post_pad, seg_out, counters);
    } else {
        launch(align_count_kernel<0>, grid, blk, 0, s, ids, numel, E, unit_hist, group_hist);
        launch(align_scatter_kernel<0>, grid, blk, 0, s, ids, numel, E, block, unit_hist, group_hist, sorted, sorted_len,
               expert_ids, eid_len, post_pad, seg_out, counters);
    }
    return launch_status();
}

int launch_align(const void* ids, int itype, int64_t numel, int E, int block,
                 int32_t* sorted, int64_t sorted_len, int32_t* expert_ids, int64_t eid_len,
                 int32_t* post_pad, int32_t* seg_out, int32_t* tickets, hipStream_t s) {
    const dim3 grid(1), blk(kAlignThreads);
    if (itype == EM_ITYPE_I32) {
        if (E == 8)
            launch((align_kernel<int32_t, 8>), grid, blk, 0, s, static_cast<const int32_t*>(ids),
                               numel, E, block, sorted, sorted_len, expert_ids, eid_len, post_pad, seg_out, tickets);
        else
            launch((align_kernel<int32_t, 0>), grid, blk, 0, s, static_cast<const int32_t*>(ids),
                               numel, E, block, sorted, sorted_len, expert_ids, eid_len, post_pad, seg_out, tickets);
    } else if (itype == EM_ITYPE_I64) {
        launch((align_kernel<int64_t, 0>), grid, blk, 0, s, static_cast<const int64_t*>(ids),
                           numel, E, block, sorted, sorted_len, expert_ids, eid_len, post_pad, seg_out, tickets);
    } else {
        return EM_ERR_BAD_DTYPE;
    }
    return launch_status();
}

bool route_align_supported(int64_t T, int E, int k) { return E == 8 && T > 0 && T * k <= kFusedMaxSlots; }

int launch_route_align(const void* logits, int logits_dtype, int64_t T, int k, int renorm, float* w, int32_t* ids,
                       int block, int32_t* sorted, int64_t sorted_len, int32_t* expert_ids, int64_t eid_len,
                       int32_t* post_pad, int32_t* seg_out, int32_t* counters, hipStream_t s) {
    const dim3 grid(1), blk(kAlignThreads);
    auto go = [&](auto kernel, auto* lp) {
        launch(kernel, grid, blk, 0, s, lp, T, k, renorm, w, ids, block, sorted, sorted_len, expert_ids,
                           eid_len, post_pad, seg_out, counters);
    };
    switch (logits_dtype) {
        case EM_DTYPE_F32: go(route_align_kernel<F32Elem>, static_cast<const F32Elem::storage*>(logits)); break;
        case EM_DTYPE_BF16: go(route_align_kernel<BF16Elem>, static_cast<const BF16Elem::storage*>(logits)); break;
        case EM_DTYPE_F16: go(route_align_kernel<F16Elem>, static_cast<const F16Elem::storage*>(logits)); break;
        default: return EM_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace em
