// Inverse neighbour index: for every vertex m the flat slots v*K+n of the
// neighbour table that name m, ascending. Every gather-instead-of-atomics kernel
// of the library reads it (gradient of the accumulation,
// modules/compiled/accumulate_knn_grad_kernel.cc:36-97; push_knn_kernel.cc:40-62;
// select_knn_grad_kernel.cu.cc:124-164 scatter with atomicAdd where this library
// gathers in a fixed order).
//
// It is a stable sort of the N*K slots by their target: the two-level counting
// sort of split_sort.hip with the table itself as the key array. Slots without a
// neighbour (index < 0 or >= N) end up behind the last vertex's list. Tables with
// 2^22 vertices and more (more tiles than the counters of a workgroup hold) take a
// library radix sort instead.
#include "hgc_common.hpp"

#include <algorithm>
#include <cstring>

#include <rocprim/rocprim.hpp>

namespace hgc {
namespace {

struct InverseKey {
    unsigned n_vert;
    __host__ __device__ unsigned operator()(int j) const { return (unsigned)j < n_vert ? (unsigned)j : n_vert; }
};

__global__ __launch_bounds__(256) void inverse_offsets_kernel(const unsigned int *__restrict__ sorted_keys,
                                                              long long total, int *__restrict__ offsets, int n_vert) {
    const int m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m > n_vert) return;
    long long lo = 0, hi = total;  // first position whose key is >= m
    while (lo < hi) {
        long long mid = (lo + hi) >> 1;
        if (sorted_keys[mid] < (unsigned)m)
            lo = mid + 1;
        else
            hi = mid;
    }
    offsets[m] = (int)lo;
}

int inverse_key_bits(int n_vert) {
    int bits = 1;
    while (bits < 32 && (1ll << bits) <= (long long)n_vert) ++bits;  // keys go up to n_vert inclusive
    return bits;
}

size_t library_sort_bytes(size_t total, int n_vert) {
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, rocprim::make_transform_iterator((const int *)nullptr, InverseKey{1u}),
                                    (unsigned int *)nullptr, rocprim::counting_iterator<int>(0), (int *)nullptr, total, 0,
                                    inverse_key_bits(std::max(n_vert, 1)), (hipStream_t) nullptr);
    return align_up(temp) + align_up(total * sizeof(int));
}

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" {

size_t hgc_inverse_neighbour_index_workspace_bytes(int n_vert, int n_neigh) {
    const size_t total = std::max<size_t>((size_t)std::max(n_vert, 0) * std::max(n_neigh, 0), 1);
    if (stable_key_sort_supported((long long)total, std::max(n_vert, 1), n_neigh))
        return stable_key_sort_workspace_bytes((long long)total, std::max(n_vert, 1), n_neigh);
    return library_sort_bytes(total, n_vert);
}

int hgc_inverse_neighbour_index(const int *d_idxs, int n_vert, int n_neigh, int *d_inv_offsets, int *d_inv_slots,
                                void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1, "bad sizes");
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neigh overflows int32");
    HGC_REQUIRE(d_inv_offsets, "null pointer");
    hipStream_t s = as_stream(stream);
    if (n_vert == 0) return launch_fill_i32(d_inv_offsets, 0, 1, s);
    HGC_REQUIRE(d_idxs && d_inv_slots, "null pointer");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_inverse_neighbour_index_workspace_bytes(n_vert, n_neigh))
        return fail(HGC_ERR_WORKSPACE, "inverse_neighbour_index workspace missing, misaligned or too small");
    const long long total = (long long)n_vert * n_neigh;
    if (stable_key_sort_supported(total, n_vert, n_neigh))
        return stable_key_sort(d_idxs, nullptr, total, n_vert, n_neigh, d_inv_offsets, d_inv_slots, workspace,
                               workspace_bytes, s);

    // Keys and values are generated on the fly: key = the slot's target (invalid
    // ones sort last), value = the flat slot itself. Stable: inside one target the
    // flat slots stay ascending, i.e. (vertex, slot) order.
    Carver carve(workspace);
    unsigned int *keys_sorted = carve.take<unsigned int>(total);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    const auto keys_in = rocprim::make_transform_iterator(d_idxs, InverseKey{(unsigned)n_vert});
    const rocprim::counting_iterator<int> slots_in(0);
    HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_sorted, slots_in, d_inv_slots, (size_t)total, 0,
                                      inverse_key_bits(n_vert), s));
    inverse_offsets_kernel<<<ceil_div((long long)n_vert + 1, 256), 256, 0, s>>>(keys_sorted, total, d_inv_offsets, n_vert);
    return check_launch("inverse_offsets");
}

}  // extern "C"
