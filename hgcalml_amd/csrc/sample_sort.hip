// Ascending sort of 64-bit keys that differ pairwise, in four launches whatever
// the distribution of the keys: the selection order of the condensate assignment
// (modules/compiled/binned_assign_to_condensates_kernel.cc:187-236 finds the next
// condensation point by a linear arg-max over beta, again and again; here the
// order of those picks is one sort by (event, class, beta descending, position)).
//
// A radix sort pays one pass per 8 key bits, each pass a few launches of a few
// microseconds on half a million keys. This one is a sample sort:
//   1. one workgroup sorts 4096 regularly spaced keys and keeps every
//      (4096 / buckets)-th as a splitter;
//   2. every key finds its bucket by binary search over the splitters (LDS),
//      workgroups count into an LDS histogram and add it to the global one;
//   3. same search again, now every workgroup reserves room in each bucket with one
//      atomic per bucket it touches and moves its keys there (the order inside a
//      bucket does not matter: its keys are sorted next);
//   4. one workgroup per bucket sorts its keys and writes the low bits of every
//      key, the payload, to its final position.
// The sorts of 1 and 4 are bitonic networks over keys in registers (1, 2, 4 or 8
// per thread of a 1024-thread workgroup): compare-exchange steps inside a thread,
// between lanes (ds_bpermute) and, for the few steps across waves, through LDS.
// Buckets hold ~2000 keys; with eight or more sampled keys per bucket one four
// times that size is out of reach for keys in any order that was not built
// against the sampling positions. A bucket beyond 8192 keys is still sorted: runs
// of that size, then pairwise merges through global memory by the same workgroup
// (slow, never seen on real inputs, exercised by the tests through a smaller run
// size).
#include "hgc_common.hpp"

#include <algorithm>

namespace hgc {
namespace {

constexpr int kSortBlock = 1024;     // threads of the workgroups that sort in LDS
constexpr int kSample = 4096;        // keys looked at for the splitters
constexpr int kBucketTarget = 2048;  // wanted keys per bucket
constexpr int kBucketStage = 8192;   // keys of a bucket that are sorted in LDS at once
constexpr int kMaxBuckets = 512;     // at least eight sampled keys per bucket
constexpr int kMoveBlock = 256;      // threads of the counting and moving kernels
constexpr int kMoveItems = 8;        // keys per thread there
constexpr uint64_t kPadKey = ~0ull;  // sorts behind every real key

__device__ __forceinline__ uint64_t key_from_lane(uint64_t v, int src_lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)(uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// one side of a compare-exchange: the smaller (keep_min) or the larger of the two keys
__device__ __forceinline__ uint64_t pick(uint64_t mine, uint64_t other, bool keep_min) {
    return ((other < mine) == keep_min) ? other : mine;
}

// Ascending bitonic sort of E * 1024 keys held in registers by the 1024 threads of a
// workgroup, thread t holding positions t*E .. t*E+E-1. A compare-exchange step at
// distance j runs inside the thread's registers (j < E), between the lanes of a wave
// (j < 64 E, ds_bpermute) or through LDS (`exchange`, E * 1024 keys laid out
// [register][thread]); of the 78 steps for 4096 keys only 10 are of the last kind.
template <int E>
__device__ __forceinline__ void block_sort_keys(uint64_t (&key)[E], uint64_t *exchange, int tid) {
    constexpr int size = E * kSortBlock;
    const int lane = tid & (kWave - 1);
    for (int k = 2; k <= size; k <<= 1) {
        int j = k >> 1;
        for (; j >= E * kWave; j >>= 1) {
            const int dt = j / E;  // the partner thread is tid ^ dt
#pragma unroll
            for (int e = 0; e < E; ++e) exchange[e * kSortBlock + tid] = key[e];
            __syncthreads();
            const bool lower = (tid & dt) == 0;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const bool up = ((tid * E + e) & k) == 0;
                key[e] = pick(key[e], exchange[e * kSortBlock + (tid ^ dt)], lower == up);
            }
            __syncthreads();
        }
        for (; j >= E; j >>= 1) {
            const int d = j / E;  // the partner lane is lane ^ d
            const bool lower = (lane & d) == 0;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const bool up = ((tid * E + e) & k) == 0;
                key[e] = pick(key[e], key_from_lane(key[e], lane ^ d), lower == up);
            }
        }
#pragma unroll
        for (int jj = E / 2; jj >= 1; jj >>= 1) {
            if (jj > (k >> 1)) continue;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                if (e & jj) continue;
                const bool up = ((tid * E + e) & k) == 0;
                const uint64_t a = key[e], b = key[e | jj];
                if ((a > b) == up) key[e] = b, key[e | jj] = a;
            }
        }
    }
}

// loads m <= E * 1024 keys (the rest: pad keys), sorts them
template <int E>
__device__ __forceinline__ void load_and_sort(const uint64_t *in, int m, uint64_t (&key)[E], uint64_t *exchange, int tid) {
#pragma unroll
    for (int e = 0; e < E; ++e) key[e] = tid * E + e < m ? in[tid * E + e] : kPadKey;
    block_sort_keys<E>(key, exchange, tid);
}

// number of splitters <= key
__device__ __forceinline__ int bucket_of(const uint64_t *splitters, int n_buckets, uint64_t key) {
    int lo = 0, hi = n_buckets - 1;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (splitters[mid] <= key)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(kSortBlock) void splitters_kernel(const uint64_t *__restrict__ keys, int n, int n_buckets,
                                                               uint64_t *__restrict__ splitters, int *__restrict__ hist,
                                                               int *__restrict__ cursor) {
    constexpr int E = kSample / kSortBlock;
    __shared__ uint64_t s_exchange[kSample];
    const int tid = threadIdx.x;
    uint64_t key[E];
#pragma unroll
    for (int e = 0; e < E; ++e) key[e] = keys[((long long)(tid * E + e) * n + n / 2) / kSample];
    for (int t = tid; t < kMaxBuckets; t += kSortBlock) hist[t] = 0, cursor[t] = 0;
    block_sort_keys<E>(key, s_exchange, tid);
    const int every = kSample / n_buckets;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int at = tid * E + e;
        if (at > 0 && at % every == 0) splitters[at / every - 1] = key[e];
    }
}

__global__ __launch_bounds__(kMoveBlock) void bucket_count_kernel(const uint64_t *__restrict__ keys, int n, int n_buckets,
                                                                  const uint64_t *__restrict__ splitters,
                                                                  int *__restrict__ hist) {
    __shared__ uint64_t s_split[kMaxBuckets];
    __shared__ int s_count[kMaxBuckets];
    const int tid = threadIdx.x;
    for (int t = tid; t < n_buckets; t += kMoveBlock) {
        s_count[t] = 0;
        if (t < n_buckets - 1) s_split[t] = splitters[t];
    }
    __syncthreads();
    const long long base = (long long)blockIdx.x * (kMoveBlock * kMoveItems);
#pragma unroll
    for (int j = 0; j < kMoveItems; ++j) {
        const long long i = base + j * kMoveBlock + tid;
        if (i < n) atomicAdd(&s_count[bucket_of(s_split, n_buckets, keys[i])], 1);
    }
    __syncthreads();
    for (int t = tid; t < n_buckets; t += kMoveBlock)
        if (s_count[t]) atomicAdd(&hist[t], s_count[t]);
}

__global__ __launch_bounds__(kMoveBlock) void bucket_move_kernel(const uint64_t *__restrict__ keys, int n, int n_buckets,
                                                                 const uint64_t *__restrict__ splitters,
                                                                 const int *__restrict__ hist, int *__restrict__ cursor,
                                                                 uint64_t *__restrict__ bucketed) {
    __shared__ uint64_t s_split[kMaxBuckets];
    __shared__ int s_count[kMaxBuckets], s_base[kMaxBuckets];
    __shared__ int s_wave_total[kMoveBlock / kWave];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;

    // where every bucket starts: exclusive sums of the histogram, two buckets per thread
    constexpr int per = kMaxBuckets / kMoveBlock;
    int h[per], mine = 0;
#pragma unroll
    for (int u = 0; u < per; ++u) {
        const int b = tid * per + u;
        h[u] = b < n_buckets ? hist[b] : 0;
        mine += h[u];
    }
    const int upto = wave_inclusive_sum(mine);
    if (lane == kWave - 1) s_wave_total[wave] = upto;
    for (int t = tid; t < n_buckets; t += kMoveBlock) {
        s_count[t] = 0;
        if (t < n_buckets - 1) s_split[t] = splitters[t];
    }
    __syncthreads();
    int before = upto - mine;
    for (int w = 0; w < wave; ++w) before += s_wave_total[w];
#pragma unroll
    for (int u = 0; u < per; ++u) {
        s_base[tid * per + u] = before;
        before += h[u];
    }
    __syncthreads();

    // this workgroup's keys: bucket, and rank among the workgroup's keys of that bucket
    const long long base = (long long)blockIdx.x * (kMoveBlock * kMoveItems);
    uint64_t key[kMoveItems];
    int bucket[kMoveItems], rank[kMoveItems];
#pragma unroll
    for (int j = 0; j < kMoveItems; ++j) {
        const long long i = base + j * kMoveBlock + tid;
        bucket[j] = -1;
        if (i < n) {
            key[j] = keys[i];
            bucket[j] = bucket_of(s_split, n_buckets, key[j]);
            rank[j] = atomicAdd(&s_count[bucket[j]], 1);
        }
    }
    __syncthreads();
    // room in every bucket this workgroup adds to
    for (int t = tid; t < n_buckets; t += kMoveBlock) {
        const int c = s_count[t];
        if (c) s_base[t] += atomicAdd(&cursor[t], c);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kMoveItems; ++j)
        if (bucket[j] >= 0) bucketed[s_base[bucket[j]] + rank[j]] = key[j];
}

// sorts m <= E * 1024 keys of `in` and hands (position, key) of the first m to `emit`
template <int E, typename Emit>
__device__ __forceinline__ void sort_run(const uint64_t *in, int m, uint64_t *exchange, int tid, Emit emit) {
    uint64_t key[E];
    load_and_sort<E>(in, m, key, exchange, tid);
#pragma unroll
    for (int e = 0; e < E; ++e)
        if (tid * E + e < m) emit(tid * E + e, key[e]);
}

template <typename Emit>
__device__ __forceinline__ void sort_run_of(const uint64_t *in, int m, uint64_t *exchange, int tid, Emit emit) {
    if (m <= kSortBlock)
        sort_run<1>(in, m, exchange, tid, emit);
    else if (m <= 2 * kSortBlock)
        sort_run<2>(in, m, exchange, tid, emit);
    else if (m <= 4 * kSortBlock)
        sort_run<4>(in, m, exchange, tid, emit);
    else
        sort_run<8>(in, m, exchange, tid, emit);
}

// One workgroup per bucket. Up to `stage` <= kBucketStage keys are sorted at once
// (smaller than the LDS array only where a test wants the path for larger
// buckets). `spare` is a second array of the keys' size.
__global__ __launch_bounds__(kSortBlock) void bucket_sort_kernel(uint64_t *bucketed, uint64_t *spare,
                                                                 const int *__restrict__ hist, int n_buckets, int n,
                                                                 int stage, uint64_t value_mask,
                                                                 int *__restrict__ values_out) {
    __shared__ uint64_t s_exchange[kBucketStage];
    __shared__ int s_start;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int b = blockIdx.x;
    int start = 0, count = n;
    if (n_buckets > 1) {
        if (tid == 0) s_start = 0;
        __syncthreads();
        int part = 0;
        for (int t = tid; t < b; t += kSortBlock) part += hist[t];
        part = wave_inclusive_sum(part);
        if (lane == kWave - 1 && part) atomicAdd(&s_start, part);
        __syncthreads();
        start = s_start;
        count = hist[b];
    }
    if (count == 0) return;

    if (count <= stage) {
        int *out = values_out + start;
        sort_run_of(bucketed + start, count, s_exchange, tid,
                    [=](int at, uint64_t key) { out[at] = (int)(key & value_mask); });
        return;
    }

    // A bucket beyond the stage: sorted runs of `stage` keys in place ...
    for (int run = 0; run < count; run += stage) {
        uint64_t *keys = bucketed + start + run;
        sort_run_of(keys, min(stage, count - run), s_exchange, tid, [=](int at, uint64_t key) { keys[at] = key; });
    }
    // ... then merged pairwise, every thread placing the output positions it owns:
    // of the r smallest keys of runs A and B, i come from A, where i is the first
    // split with A[i] >= B[r - i - 1].
    uint64_t *src = bucketed + start, *dst = spare + start;
    for (long long width = stage; width < count; width *= 2) {
        __threadfence();  // the other waves' keys of the last pass
        __syncthreads();
        for (int o = tid; o < count; o += kSortBlock) {
            const int a0 = (int)(o / (2 * width) * (2 * width));
            const int a_len = (int)min(width, (long long)count - a0);
            const int b0 = a0 + a_len;
            const int b_len = (int)min(width, (long long)count - b0);
            const int r = o - a0;
            int lo = max(0, r - b_len), hi = min(r, a_len);
            while (lo < hi) {
                const int i = (lo + hi) >> 1;
                if (src[a0 + i] < src[b0 + (r - i - 1)])
                    lo = i + 1;
                else
                    hi = i;
            }
            const int i = lo, j = r - lo;
            const bool from_a = i < a_len && (j >= b_len || src[a0 + i] < src[b0 + j]);
            dst[o] = from_a ? src[a0 + i] : src[b0 + j];
        }
        uint64_t *t = src;
        src = dst;
        dst = t;
    }
    __threadfence();
    __syncthreads();
    for (int o = tid; o < count; o += kSortBlock) values_out[start + o] = (int)(src[o] & value_mask);
}

int buckets_for(long long n) {
    if (n <= kBucketStage) return 1;
    int buckets = 2;
    while ((long long)buckets * kBucketTarget < n && buckets < kMaxBuckets) buckets <<= 1;
    return buckets;
}

}  // namespace

bool sample_sort_supported(long long n) { return n >= 0 && n <= (long long)kMaxBuckets * kBucketTarget; }

size_t sample_sort_workspace_bytes() {
    return align_up(kMaxBuckets * sizeof(uint64_t)) + 2 * align_up(kMaxBuckets * sizeof(int));
}

// Sorts d_keys[0, n) (pairwise different, none of them all ones; overwritten) and
// writes the low `value_bits` bits of the i-th smallest key to d_values[i].
// d_spare: n more keys. `stage` = 0, or the number of keys sorted in LDS at once
// (a power of two up to 8192; tests use a small one).
int sample_sort_values(uint64_t *d_keys, uint64_t *d_spare, long long n, int value_bits, int *d_values,
                       void *workspace, size_t workspace_bytes, int stage, hipStream_t s) {
    HGC_REQUIRE(sample_sort_supported(n), "sample sort: too many keys");
    HGC_REQUIRE(value_bits >= 1 && value_bits <= 31, "sample sort: 1 <= value bits <= 31");
    if (stage == 0) stage = kBucketStage;
    HGC_REQUIRE(stage >= 2 && stage <= kBucketStage && (stage & (stage - 1)) == 0, "sample sort: bad stage");
    if (n == 0) return HGC_OK;
    HGC_REQUIRE(d_keys && d_spare && d_values, "null pointer");
    if (!workspace || !aligned256(workspace) || workspace_bytes < sample_sort_workspace_bytes())
        return fail(HGC_ERR_WORKSPACE, "sample sort workspace missing, misaligned or too small");
    const uint64_t mask = (1ull << value_bits) - 1ull;
    const int buckets = buckets_for(n);
    if (buckets == 1) {
        bucket_sort_kernel<<<1, kSortBlock, 0, s>>>(d_keys, d_spare, nullptr, 1, (int)n, stage, mask, d_values);
        return check_launch("bucket_sort");
    }
    Carver carve(workspace);
    uint64_t *splitters = carve.take<uint64_t>(kMaxBuckets);
    int *hist = carve.take<int>(kMaxBuckets);
    int *cursor = carve.take<int>(kMaxBuckets);
    int rc;
    splitters_kernel<<<1, kSortBlock, 0, s>>>(d_keys, (int)n, buckets, splitters, hist, cursor);
    if ((rc = check_launch("splitters"))) return rc;
    const int blocks = (int)ceil_div(n, (long long)kMoveBlock * kMoveItems);
    bucket_count_kernel<<<blocks, kMoveBlock, 0, s>>>(d_keys, (int)n, buckets, splitters, hist);
    if ((rc = check_launch("bucket_count"))) return rc;
    bucket_move_kernel<<<blocks, kMoveBlock, 0, s>>>(d_keys, (int)n, buckets, splitters, hist, cursor, d_spare);
    if ((rc = check_launch("bucket_move"))) return rc;
    // the buckets sit in d_spare; the input array is the second array of the merges
    bucket_sort_kernel<<<buckets, kSortBlock, 0, s>>>(d_spare, d_keys, hist, buckets, (int)n, stage, mask, d_values);
    return check_launch("bucket_sort");
}

}  // namespace hgc

using namespace hgc;

extern "C" {

size_t hgc_sort_distinct_keys_workspace_bytes(long long n) {
    return align_up((size_t)std::max(n, 1ll) * sizeof(uint64_t)) + sample_sort_workspace_bytes();
}

int hgc_sort_distinct_keys(unsigned long long *d_keys, long long n, int value_bits, int *d_values, void *workspace,
                           size_t workspace_bytes, int stage, hgc_stream_t stream) {
    HGC_REQUIRE(n >= 0 && sample_sort_supported(n), "0 <= n <= 2^20");
    if (!workspace || !aligned256(workspace) || workspace_bytes < hgc_sort_distinct_keys_workspace_bytes(n))
        return fail(HGC_ERR_WORKSPACE, "sort_distinct_keys workspace missing, misaligned or too small");
    Carver carve(workspace);
    uint64_t *spare = carve.take<uint64_t>((size_t)std::max(n, 1ll));
    return sample_sort_values(reinterpret_cast<uint64_t *>(d_keys), spare, n, value_bits, d_values,
                              carve.base + carve.used, workspace_bytes - carve.used, stage, as_stream(stream));
}

}  // extern "C"
