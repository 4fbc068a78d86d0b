// Expert-centric bucketing for gfx950: (token, k) pairs grouped by expert id.
//
//   histogram   counts[e] = number of pairs with id e                     (integer atomics: order-independent)
//   scan        offsets[e] = sum of counts[< e], offsets[E] = number of valid pairs; one pass, any number of
//               workgroups (tiles are taken by ticket; a tile publishes its total, then adds up its predecessors)
//   fill        sorted_pairs[offsets[e] + arrival] = p for every pair p of expert e
//   order       each segment put in ascending pair index (what a stable sort by expert id gives), so that the
//               result does not depend on the order in which the fill's atomics were served
//
// Ids outside [0, E) belong to no segment.  This is the on-GPU form of the sort / bincount / cumsum preprocessing of
// the reference (flash_moe/ops/triton/flash_expert.py:528-577), without its host synchronisation.
#include "fmoe_common.h"

namespace fmoe {
namespace {

constexpr int kScanThreads = 1024;
constexpr int kScanTile = kScanThreads * 4;
constexpr uint64_t kFlagAggregate = 1ull << 32, kFlagInclusive = 2ull << 32;

__global__ __launch_bounds__(256) void bucket_clear_kernel(int32_t* __restrict__ p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

__global__ __launch_bounds__(256) void bucket_histogram_kernel(const int64_t* __restrict__ indices, int32_t* __restrict__ counts,
                                                               int64_t num_pairs, int64_t num_experts) {
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < num_pairs; p += (int64_t)gridDim.x * blockDim.x) {
        const int64_t e = indices[p];
        if (e >= 0 && e < num_experts) atomicAdd(&counts[e], 1);
    }
}

__device__ inline void publish(uint64_t* slot, uint64_t v) {
    __hip_atomic_store(slot, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline uint64_t peek(uint64_t* slot) {
    return __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// counts[e] is replaced by offsets[e] (the fill's running cursor of expert e); offsets[0..E] is the result.
// A workgroup takes the next tile by ticket, so every tile before it is already running (or done) when it waits for
// that tile's total: the wait always ends.  status[t] = flag << 32 | value, one 64-bit word per tile.
__global__ __launch_bounds__(kScanThreads) void bucket_scan_kernel(int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                                  int64_t num_experts, int32_t* __restrict__ ticket,
                                                                  uint64_t* __restrict__ status) {
    __shared__ int32_t wave_total[kScanThreads / kWave];
    __shared__ int32_t tile_s, before_s;
    const int tid = (int)threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    if (tid == 0) tile_s = atomicAdd(ticket, 1);
    __syncthreads();
    const int tile = tile_s;
    const int64_t e0 = (int64_t)tile * kScanTile + (int64_t)tid * 4;
    int32_t c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = e0 + j < num_experts ? counts[e0 + j] : 0;
    const int32_t mine = c[0] + c[1] + c[2] + c[3];
    int32_t incl = mine;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int32_t up = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_total[wave] = incl;
    __syncthreads();
    if (tid == 0) {
        int32_t total = 0;
        for (int w = 0; w < kScanThreads / kWave; ++w) total += wave_total[w];
        int32_t before = 0;
        if (tile > 0) {
            publish(&status[tile], kFlagAggregate | (uint32_t)total);
            for (int j = tile - 1; j >= 0; --j) {
                uint64_t s;
                do { s = peek(&status[j]); } while ((s >> 32) == 0);
                before += (int32_t)(uint32_t)s;
                if (s & kFlagInclusive) break;
            }
        }
        publish(&status[tile], kFlagInclusive | (uint32_t)(before + total));
        before_s = before;
        if ((int64_t)(tile + 1) * kScanTile >= num_experts) offsets[num_experts] = before + total;   // the last tile
    }
    __syncthreads();
    int32_t run = before_s + incl - mine;
    for (int w = 0; w < wave; ++w) run += wave_total[w];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (e0 + j < num_experts) {
            offsets[e0 + j] = run;
            counts[e0 + j] = run;
        }
        run += c[j];
    }
}

// Pair p of expert e goes to slot cursor[e]++.  tok[slot] = token * tok_scale and exp[slot] = e * exp_scale are what the
// consumers index with (ids with scale 1, row byte offsets otherwise).  A pair with an id outside [0,E) belongs to no
// segment: its entry of `coef_clear` (optional, [num_pairs]) is zeroed so that a later pass over all pairs reads a
// defined value, and when `tail` is given it zeroes one of the slots after the last segment (offsets[E] + a ticket from
// the counter `tail`), so that tok and exp are defined over all num_pairs slots.
__global__ __launch_bounds__(256) void bucket_fill_kernel(const int64_t* __restrict__ indices, int32_t* __restrict__ cursor,
                                                          int32_t* __restrict__ sorted_pairs, uint32_t* __restrict__ tok,
                                                          uint32_t* __restrict__ exp, float* __restrict__ coef_clear,
                                                          const int32_t* __restrict__ offsets, int32_t* __restrict__ tail,
                                                          int64_t num_pairs, int64_t num_experts, int top_k,
                                                          uint32_t tok_scale, uint32_t exp_scale, int pack_shift) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= num_pairs) return;
    const int64_t e = indices[p];
    if (e < 0 || e >= num_experts) {
        if (coef_clear != nullptr) coef_clear[p] = 0.0f;
        if (tail != nullptr) {
            const int32_t slot = offsets[num_experts] + atomicAdd(tail, 1);
            if (tok != nullptr) tok[slot] = 0u;
            if (exp != nullptr) exp[slot] = 0u;
        }
        return;
    }
    const int32_t slot = atomicAdd(&cursor[e], 1);
    sorted_pairs[slot] = (int32_t)p;
    // pack_shift: the low bits of the id ride in the token word above that bit (token | (e << shift), truncated)
    if (tok != nullptr) tok[slot] = (uint32_t)(p / top_k) * tok_scale | (pack_shift ? (uint32_t)e << pack_shift : 0u);
    if (exp != nullptr) exp[slot] = (uint32_t)e * exp_scale;
}

// ---- ascending pair index inside every segment -------------------------------------------------------------------
constexpr int kOrderWaves = 4;
constexpr int kOrderLds = 4096;      // longest segment sorted in LDS

// Four experts per workgroup.  Segments of up to 64 pairs: one wave each, rank by counting.  Up to kOrderLds: the
// workgroup, bitonic network in LDS.  Longer: the workgroup walks the whole index array in order and writes the
// expert's pairs as it meets them (a stable compaction; cost proportional to the number of pairs, for experts that a
// large share of all tokens selected).
__global__ __launch_bounds__(kOrderWaves* kWave) void bucket_order_kernel(
    const int64_t* __restrict__ indices, const int32_t* __restrict__ offsets, int32_t* __restrict__ sorted_pairs,
    uint32_t* __restrict__ tok, int64_t num_pairs, int64_t num_experts, int top_k, uint32_t tok_scale) {
    __shared__ uint32_t keys[kOrderLds];
    __shared__ int32_t wave_count[4][kOrderWaves];
    const int tid = (int)threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int64_t e_first = (int64_t)blockIdx.x * kOrderWaves;
    {
        const int64_t e = e_first + wave;
        if (e < num_experts) {
            const int begin = __builtin_amdgcn_readfirstlane(offsets[e]);
            const int n = __builtin_amdgcn_readfirstlane(offsets[e + 1]) - begin;
            if (n > 1 && n <= kWave) {
                const uint32_t p = lane < n ? (uint32_t)sorted_pairs[begin + lane] : 0xFFFFFFFFu;
                int rank = 0;
                for (int j = 0; j < n; ++j) rank += ((uint32_t)__builtin_amdgcn_readlane((int)p, j) < p) ? 1 : 0;
                if (lane < n) {
                    sorted_pairs[begin + rank] = (int32_t)p;
                    if (tok != nullptr) tok[begin + rank] = (p / (uint32_t)top_k) * tok_scale;
                }
            }
        }
    }
    for (int w = 0; w < kOrderWaves; ++w) {
        const int64_t e = e_first + w;
        if (e >= num_experts) break;
        const int begin = offsets[e], n = offsets[e + 1] - begin;      // the same for every thread of the workgroup
        if (n <= kWave) continue;
        __syncthreads();
        if (n <= kOrderLds) {
            int m = 128;
            while (m < n) m <<= 1;
            for (int i = tid; i < m; i += kOrderWaves * kWave) keys[i] = i < n ? (uint32_t)sorted_pairs[begin + i] : 0xFFFFFFFFu;
            __syncthreads();
            for (int k = 2; k <= m; k <<= 1)
                for (int j = k >> 1; j > 0; j >>= 1) {
                    for (int i = tid; i < m / 2; i += kOrderWaves * kWave) {
                        const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1)), hi = lo | j;
                        const uint32_t a = keys[lo], b = keys[hi];
                        const bool ascending = (lo & k) == 0;
                        if ((a > b) == ascending) {
                            keys[lo] = b;
                            keys[hi] = a;
                        }
                    }
                    __syncthreads();
                }
            for (int i = tid; i < n; i += kOrderWaves * kWave) {
                sorted_pairs[begin + i] = (int32_t)keys[i];
                if (tok != nullptr) tok[begin + i] = (keys[i] / (uint32_t)top_k) * tok_scale;
            }
        } else {
            // kOrderBatch rounds of 256 pairs per pair of barriers: their index loads are in flight together
            constexpr int kOrderBatch = 4, kRound = kOrderWaves * kWave;
            int32_t written = 0;
            for (int64_t base = 0; base < num_pairs; base += kOrderBatch * kRound) {
                bool hit[kOrderBatch];
                uint64_t ballot[kOrderBatch];
#pragma unroll
                for (int u = 0; u < kOrderBatch; ++u) {
                    const int64_t p = base + u * kRound + tid;
                    hit[u] = p < num_pairs && indices[p] == e;
                }
#pragma unroll
                for (int u = 0; u < kOrderBatch; ++u) {
                    ballot[u] = __ballot(hit[u]);
                    if (lane == 0) wave_count[u][wave] = __popcll(ballot[u]);
                }
                __syncthreads();
#pragma unroll
                for (int u = 0; u < kOrderBatch; ++u) {
                    int32_t before = written, all = 0;
                    for (int v = 0; v < kOrderWaves; ++v) {
                        if (v < wave) before += wave_count[u][v];
                        all += wave_count[u][v];
                    }
                    if (hit[u]) {
                        const int64_t p = base + u * kRound + tid;
                        const int32_t slot = begin + before + __popcll(ballot[u] & ((1ull << lane) - 1ull));
                        sorted_pairs[slot] = (int32_t)p;
                        if (tok != nullptr) tok[slot] = (uint32_t)(p / top_k) * tok_scale;
                    }
                    written += all;
                }
                __syncthreads();
            }
        }
    }
}

// ---- grouping by two partition passes --------------------------------------------------------------------------------
// For millions of pairs the histogram and the fill above are bound by the rate of global atomics (20-28 G/s) and by
// scattered 4-byte writes.  Here no global atomic is issued: the pairs are first partitioned into at most 1024 coarse
// buckets of 2^shift consecutive experts (per tile of pairs a histogram in LDS, one scan over (bucket, tile), then each tile
// writes its pairs behind its own offsets), and one workgroup per coarse bucket finishes it in LDS (counts per expert,
// scan = the expert offsets, slots handed out by LDS cursors).  Pairs with an id outside [0, E) form one more bucket at the
// end, whose slots are the zeroed tail.  The order inside an expert's segment is whatever the LDS serves first.
// pairs per workgroup of the partition passes: long runs per (tile, bucket) for millions of pairs, more workgroups for fewer
inline int partition_tile(int64_t num_pairs) { return num_pairs >= (1ll << 21) ? 8192 : 2048; }
constexpr int kPartMaxBuckets = 1024;    // coarse buckets, not counting the one for invalid ids
constexpr int kPartMaxShift = 13;        // 2^13 experts per coarse bucket: 32 KiB of LDS counters

__global__ __launch_bounds__(256) void partition_count_kernel(const int64_t* __restrict__ indices, int32_t* __restrict__ counts1,
                                                              int64_t num_pairs, int64_t num_experts, int shift, int buckets,
                                                              int groups, int tile, int32_t* __restrict__ ticket,
                                                              uint64_t* __restrict__ status, int tiles) {
    __shared__ int32_t hist[kPartMaxBuckets + 1];
    const int g = (int)blockIdx.x, tid = (int)threadIdx.x;
    if (g == 0) {      // the state of the scan that follows
        if (tid == 0) *ticket = 0;
        for (int i = tid; i < tiles; i += 256) status[i] = 0;
    }
    for (int b = tid; b <= buckets; b += 256) hist[b] = 0;
    __syncthreads();
    const int64_t p0 = (int64_t)g * tile;
    for (int i = tid; i < tile; i += 256) {
        const int64_t p = p0 + i;
        if (p < num_pairs) {
            const int64_t e = indices[p];
            atomicAdd(&hist[(e >= 0 && e < num_experts) ? (int)(e >> shift) : buckets], 1);
        }
    }
    __syncthreads();
    for (int b = tid; b <= buckets; b += 256) counts1[(int64_t)b * groups + g] = hist[b];
}

// stage[slot] = pair index << 32 | id inside its coarse bucket (all ones for an invalid id)
__global__ __launch_bounds__(256) void partition_scatter_kernel(const int64_t* __restrict__ indices,
                                                                const int32_t* __restrict__ offs1, uint64_t* __restrict__ stage,
                                                                float* __restrict__ coef_clear, int64_t num_pairs,
                                                                int64_t num_experts, int shift, int buckets, int groups,
                                                                int tile) {
    __shared__ int32_t base[kPartMaxBuckets + 1];
    const int g = (int)blockIdx.x, tid = (int)threadIdx.x;
    for (int b = tid; b <= buckets; b += 256) base[b] = offs1[(int64_t)b * groups + g];
    __syncthreads();
    const int64_t p0 = (int64_t)g * tile;
    for (int i = tid; i < tile; i += 256) {
        const int64_t p = p0 + i;
        if (p < num_pairs) {
            const int64_t e = indices[p];
            const bool ok = e >= 0 && e < num_experts;
            const int b = ok ? (int)(e >> shift) : buckets;
            const int32_t slot = atomicAdd(&base[b], 1);
            stage[slot] = ((uint64_t)(uint32_t)p << 32) | (ok ? (uint32_t)(e - ((int64_t)b << shift)) : 0xFFFFFFFFu);
            if (!ok && coef_clear != nullptr) coef_clear[p] = 0.0f;
        }
    }
}

constexpr int kPartLocalThreads = 512;
constexpr int kPartLocalCap = 8192;      // pairs of a coarse bucket that are put in order in LDS and written out coalesced

__global__ __launch_bounds__(kPartLocalThreads) void partition_local_kernel(
    const uint64_t* __restrict__ stage, const int32_t* __restrict__ offs1, int32_t* __restrict__ offsets,
    int32_t* __restrict__ sorted_pairs, uint32_t* __restrict__ tok, uint32_t* __restrict__ exp, int64_t num_experts, int shift,
    int buckets, int groups, int top_k, uint32_t tok_scale, uint32_t exp_scale, int pack_shift) {
    extern __shared__ int32_t cnt[];     // 1 << shift
    __shared__ uint32_t out_pair[kPartLocalCap];
    __shared__ uint16_t out_low[kPartLocalCap];
    __shared__ int32_t wave_total[kPartLocalThreads / kWave];
    constexpr int NT = kPartLocalThreads;
    const int b = (int)blockIdx.x, tid = (int)threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int32_t begin = offs1[(int64_t)b * groups], end = offs1[(int64_t)(b + 1) * groups];
    if (b == buckets) {      // the slots after the last segment
        if (tid == 0) offsets[num_experts] = begin;
        for (int32_t s = begin + tid; s < end; s += NT) {
            if (tok != nullptr) tok[s] = 0u;
            if (exp != nullptr) exp[s] = 0u;
        }
        return;
    }
    const int64_t e0 = (int64_t)b << shift;
    const int n_e = (int)(num_experts - e0 < (1ll << shift) ? num_experts - e0 : (1ll << shift));
    for (int j = tid; j < n_e; j += NT) cnt[j] = 0;
    __syncthreads();
    for (int32_t s = begin + tid; s < end; s += 2 * NT) {
        const uint64_t v0 = stage[s], v1 = s + NT < end ? stage[s + NT] : 0;
        atomicAdd(&cnt[(uint32_t)v0], 1);
        if (s + NT < end) atomicAdd(&cnt[(uint32_t)v1], 1);
    }
    __syncthreads();
    // exclusive scan of the counts: thread t owns experts [t * per, (t + 1) * per)
    const int per = (n_e + NT - 1) / NT;
    const int j0 = tid * per < n_e ? tid * per : n_e, j1 = j0 + per < n_e ? j0 + per : n_e;
    int32_t mine = 0;
    for (int j = j0; j < j1; ++j) mine += cnt[j];
    int32_t incl = mine;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int32_t up = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_total[wave] = incl;
    __syncthreads();
    int32_t run = begin + incl - mine;
    for (int w = 0; w < wave; ++w) run += wave_total[w];
    for (int j = j0; j < j1; ++j) {
        const int32_t c = cnt[j];
        offsets[e0 + j] = run;
        cnt[j] = run;            // the cursor of expert e0 + j
        run += c;
    }
    __syncthreads();
    auto emit = [&](int32_t slot, uint32_t p, uint32_t low) {
        const uint32_t e = (uint32_t)e0 + low;
        sorted_pairs[slot] = (int32_t)p;
        if (tok != nullptr) tok[slot] = (p / (uint32_t)top_k) * tok_scale | (pack_shift ? e << pack_shift : 0u);
        if (exp != nullptr) exp[slot] = e * exp_scale;
    };
    const bool in_lds = end - begin <= kPartLocalCap;      // else (a few experts took a large share of all pairs): slot by slot
    for (int32_t s = begin + tid; s < end; s += 2 * NT) {
        const bool two = s + NT < end;
        const uint64_t v0 = stage[s], v1 = two ? stage[s + NT] : 0;
        const int32_t slot0 = atomicAdd(&cnt[(uint32_t)v0], 1);
        const int32_t slot1 = two ? atomicAdd(&cnt[(uint32_t)v1], 1) : 0;
        if (in_lds) {
            out_pair[slot0 - begin] = (uint32_t)(v0 >> 32);
            out_low[slot0 - begin] = (uint16_t)v0;
            if (two) {
                out_pair[slot1 - begin] = (uint32_t)(v1 >> 32);
                out_low[slot1 - begin] = (uint16_t)v1;
            }
        } else {
            emit(slot0, (uint32_t)(v0 >> 32), (uint32_t)v0);
            if (two) emit(slot1, (uint32_t)(v1 >> 32), (uint32_t)v1);
        }
    }
    if (!in_lds) return;
    __syncthreads();
    for (int32_t i = tid; i < end - begin; i += NT) emit(begin + i, out_pair[i], out_low[i]);
}

struct PartitionPlan {
    int shift, buckets, groups, tile, tiles;
    int64_t n1;
    size_t off_counts, off_offs, off_ticket, off_status, off_stage, bytes;
};
PartitionPlan plan_partition(int64_t num_pairs, int64_t num_experts) {
    PartitionPlan p;
    p.shift = 0;
    while (((num_experts + (1ll << p.shift) - 1) >> p.shift) > kPartMaxBuckets) ++p.shift;
    p.buckets = (int)((num_experts + (1ll << p.shift) - 1) >> p.shift);
    p.tile = partition_tile(num_pairs);
    p.groups = (int)((num_pairs + p.tile - 1) / p.tile);
    p.n1 = (int64_t)(p.buckets + 1) * p.groups;
    p.tiles = (int)((p.n1 + kScanTile - 1) / kScanTile);
    size_t o = 0;
    auto take = [&](size_t n) { const size_t at = o; o = round_up(o + n, 256); return at; };
    p.off_counts = take((size_t)p.n1 * 4);
    p.off_offs = take((size_t)(p.n1 + 1) * 4);
    p.off_ticket = take(256);
    p.off_status = take((size_t)p.tiles * 8);
    p.off_stage = take((size_t)num_pairs * 8);
    p.bytes = o;
    return p;
}

struct BucketPlan {
    int tiles;
    size_t off_cursor, off_ticket, off_status, bytes;
};
BucketPlan plan_bucket(int64_t num_experts) {
    BucketPlan p;
    p.tiles = (int)((num_experts + kScanTile - 1) / kScanTile);
    p.off_cursor = 0;
    p.off_ticket = round_up((size_t)num_experts * 4, 256);
    p.off_status = p.off_ticket + 256;
    p.bytes = round_up(p.off_status + (size_t)p.tiles * 8, 256);
    return p;
}

}  // namespace

size_t bucket_workspace_bytes(int64_t num_experts) { return plan_bucket(num_experts).bytes; }

// With millions of pairs the partition passes are far ahead of the atomics; with fewer both are a handful of launches
// at their floor, and below 65536 pairs the tiles would be too few to fill the chip.
bool bucket_partition_pays(int64_t num_pairs, int64_t num_experts) {
    if (num_pairs < (1ll << 16) || num_pairs >= (1ll << 31) || num_experts >= (1ll << 31) - 1) return false;
    const PartitionPlan p = plan_partition(num_pairs, num_experts);
    return p.shift <= kPartMaxShift && p.n1 < (1ll << 31) - 1;
}

size_t bucket_partition_workspace_bytes(int64_t num_pairs, int64_t num_experts) {
    return bucket_partition_pays(num_pairs, num_experts) ? plan_partition(num_pairs, num_experts).bytes : 0;
}

int bucket_partition(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, int top_k,
                     int32_t* offsets, int32_t* sorted_pairs, uint32_t* tok, uint32_t tok_scale, uint32_t* exp,
                     uint32_t exp_scale, float* coef_clear, int pack_shift, hipStream_t stream) {
    const PartitionPlan p = plan_partition(num_pairs, num_experts);
    char* ws = (char*)workspace;
    int32_t* counts1 = (int32_t*)(ws + p.off_counts);
    int32_t* offs1 = (int32_t*)(ws + p.off_offs);
    int32_t* ticket = (int32_t*)(ws + p.off_ticket);
    uint64_t* status = (uint64_t*)(ws + p.off_status);
    uint64_t* stage = (uint64_t*)(ws + p.off_stage);
    hipLaunchKernelGGL(partition_count_kernel, dim3((unsigned)p.groups), dim3(256), 0, stream, indices, counts1, num_pairs,
                       num_experts, p.shift, p.buckets, p.groups, p.tile, ticket, status, p.tiles);
    FMOE_CHECK_LAUNCH("expert bucketing (partition counts)");
    hipLaunchKernelGGL(bucket_scan_kernel, dim3((unsigned)p.tiles), dim3(kScanThreads), 0, stream, counts1, offs1, p.n1, ticket,
                       status);
    FMOE_CHECK_LAUNCH("expert bucketing (partition scan)");
    hipLaunchKernelGGL(partition_scatter_kernel, dim3((unsigned)p.groups), dim3(256), 0, stream, indices,
                       (const int32_t*)offs1, stage, coef_clear, num_pairs, num_experts, p.shift, p.buckets, p.groups, p.tile);
    FMOE_CHECK_LAUNCH("expert bucketing (partition scatter)");
    hipLaunchKernelGGL(partition_local_kernel, dim3((unsigned)(p.buckets + 1)), dim3(kPartLocalThreads), (size_t)4 << p.shift, stream,
                       (const uint64_t*)stage, (const int32_t*)offs1, offsets, sorted_pairs, tok, exp, num_experts, p.shift,
                       p.buckets, p.groups, top_k, tok_scale, exp_scale, pack_shift);
    FMOE_CHECK_LAUNCH("expert bucketing (partition local)");
    return FMOE_OK;
}

int32_t* bucket_counts(void* workspace) { return (int32_t*)workspace; }

int bucket_clear(void* workspace, int64_t num_experts, hipStream_t stream) {
    const BucketPlan p = plan_bucket(num_experts);
    const int64_t n = (int64_t)(p.bytes / 4);
    const unsigned grid = (unsigned)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
    hipLaunchKernelGGL(bucket_clear_kernel, dim3(grid), dim3(256), 0, stream, (int32_t*)workspace, n);
    FMOE_CHECK_LAUNCH("expert bucketing (clear)");
    return FMOE_OK;
}

int bucket_histogram(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, hipStream_t stream) {
    const int64_t blocks = (num_pairs + 255) / 256;
    hipLaunchKernelGGL(bucket_histogram_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream, indices,
                       bucket_counts(workspace), num_pairs, num_experts);
    FMOE_CHECK_LAUNCH("expert bucketing (histogram)");
    return FMOE_OK;
}

int bucket_scan_fill(const int64_t* indices, void* workspace, int64_t num_pairs, int64_t num_experts, int top_k,
                     int32_t* offsets, int32_t* sorted_pairs, uint32_t* tok, uint32_t tok_scale, uint32_t* exp,
                     uint32_t exp_scale, float* coef_clear, int pack_shift, int ordered, hipStream_t stream) {
    const BucketPlan p = plan_bucket(num_experts);
    char* ws = (char*)workspace;
    hipLaunchKernelGGL(bucket_scan_kernel, dim3((unsigned)p.tiles), dim3(kScanThreads), 0, stream, (int32_t*)(ws + p.off_cursor),
                       offsets, num_experts, (int32_t*)(ws + p.off_ticket), (uint64_t*)(ws + p.off_status));
    FMOE_CHECK_LAUNCH("expert bucketing (scan)");
    if (num_pairs == 0) return FMOE_OK;
    hipLaunchKernelGGL(bucket_fill_kernel, dim3((unsigned)((num_pairs + 255) / 256)), dim3(256), 0, stream, indices,
                       (int32_t*)(ws + p.off_cursor), sorted_pairs, tok, exp, coef_clear, (const int32_t*)offsets,
                       (tok != nullptr || exp != nullptr) ? (int32_t*)(ws + p.off_ticket) + 1 : nullptr, num_pairs, num_experts,
                       top_k, tok_scale, exp_scale, pack_shift);
    FMOE_CHECK_LAUNCH("expert bucketing (fill)");
    if (ordered) {
        hipLaunchKernelGGL(bucket_order_kernel, dim3((unsigned)((num_experts + kOrderWaves - 1) / kOrderWaves)),
                           dim3(kOrderWaves * kWave), 0, stream, indices, (const int32_t*)offsets, sorted_pairs, tok, num_pairs,
                           num_experts, top_k, tok_scale);
        FMOE_CHECK_LAUNCH("expert bucketing (order)");
    }
    return FMOE_OK;
}

}  // namespace fmoe

extern "C" size_t fmoe_expert_bucket_workspace_bytes(int64_t num_experts) {
    return num_experts > 0 ? fmoe::bucket_workspace_bytes(num_experts) : 0;
}

extern "C" int fmoe_expert_bucket(const int64_t* indices, int64_t num_tokens, int top_k, int64_t num_experts,
                                  int32_t* expert_offsets, int32_t* sorted_pair_ids, int32_t* sorted_token_ids,
                                  int32_t* sorted_expert_ids, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fmoe;
    clear_error();
    FMOE_REQUIRE(num_tokens >= 0 && top_k >= 0 && num_experts > 0, FMOE_ERR_BAD_SHAPE,
                 "fmoe_expert_bucket: bad shape T=%lld K=%d E=%lld", (long long)num_tokens, top_k, (long long)num_experts);
    FMOE_REQUIRE(num_experts < (1ll << 31) - 1 && num_tokens * (int64_t)top_k < (1ll << 31), FMOE_ERR_UNSUPPORTED,
                 "fmoe_expert_bucket: E=%lld or T*K=%lld >= 2^31", (long long)num_experts, (long long)num_tokens * top_k);
    FMOE_REQUIRE(expert_offsets && workspace, FMOE_ERR_NULL_POINTER, "fmoe_expert_bucket: null offsets / workspace pointer");
    const size_t need = bucket_workspace_bytes(num_experts);
    FMOE_REQUIRE(workspace_bytes >= need && aligned16(workspace), FMOE_ERR_WORKSPACE,
                 "fmoe_expert_bucket: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    const int64_t pairs = num_tokens * (int64_t)top_k;
    FMOE_REQUIRE(pairs == 0 || (indices && sorted_pair_ids), FMOE_ERR_NULL_POINTER, "fmoe_expert_bucket: null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    if (int rc = bucket_clear(workspace, num_experts, s)) return rc;
    if (pairs > 0)
        if (int rc = bucket_histogram(indices, workspace, pairs, num_experts, s)) return rc;
    // with no pairs the scan of the cleared counts still writes the all-zero offsets
    return bucket_scan_fill(indices, workspace, pairs, num_experts, top_k > 0 ? top_k : 1, expert_offsets, sorted_pair_ids,
                            (uint32_t*)sorted_token_ids, 1u, (uint32_t*)sorted_expert_ids, 1u, nullptr, 0, 1, s);
}
