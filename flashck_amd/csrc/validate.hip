// Debug aids (gfx950): a checker of the paged-cache arguments the attention kernels trust, and the reset of the fused
// split-KV entry point's arrival tickets.  Neither is on the hot path; both are single small launches that allocate
// nothing.
#include "common.hpp"
#include "kernels.hpp"

namespace fck {

// One workgroup walks every sequence and every table entry a sequence uses, counts what the kernels would not
// survive, and writes the four counters (no zeroing by the caller is needed):
//   counts[0]  sequences whose key count is negative or exceeds what their table row / page list can address
//   counts[1]  page ids outside [0, num_total_pages) among the entries the sequences use
//   counts[2]  page lists that are malformed: kv_indptr not monotone, kv_last_page_lens outside [1, page] on a
//              non-empty list
//   counts[3]  index of the first offending sequence, or -1
__global__ __launch_bounds__(256) void validate_paged_kernel(const ValidateArgs a)
{
    __shared__ int sums[3];
    __shared__ int first;
    const int tid = threadIdx.x;
    if (tid < 3) sums[tid] = 0;
    if (tid == 0) first = INT32_MAX;
    __syncthreads();
    int bad_len = 0, bad_page = 0, bad_list = 0, first_bad = INT32_MAX;
    for (int b = tid; b < a.batch; b += 256) {
        const int32_t* table;
        int64_t entries, used, len;
        bool list_ok = true;
        if (a.block_table) {
            table = a.block_table + (int64_t)b * a.block_table_stride;
            entries = a.block_table_stride;
            len = a.seqlen_k[b];
            used = len > 0 ? (len + a.page_size - 1) / a.page_size : 0;
        } else {
            const int64_t p0 = a.kv_indptr[b], p1 = a.kv_indptr[b + 1];
            table = a.kv_page_indices + p0;
            entries = p1 - p0;
            list_ok = p0 >= 0 && entries >= 0;
            const int64_t last = a.kv_last_page_lens ? a.kv_last_page_lens[b] : a.page_size;
            if (entries > 0 && (last < 1 || last > a.page_size)) list_ok = false;
            len = entries > 0 ? (entries - 1) * a.page_size + last : 0;
            used = list_ok ? entries : 0;
        }
        const bool len_ok = !list_ok || (len >= 0 && used <= entries);  // a malformed list is counted once, as that
        int pages_bad = 0;
        if (len_ok && list_ok)
            for (int64_t i = 0; i < used; ++i) {
                const int64_t p = table[i];
                pages_bad += (p < 0 || p >= a.num_total_pages) ? 1 : 0;
            }
        bad_len += len_ok ? 0 : 1;
        bad_list += list_ok ? 0 : 1;
        bad_page += pages_bad;
        if ((!len_ok || !list_ok || pages_bad) && b < first_bad) first_bad = b;
    }
    if (bad_len) atomicAdd(&sums[0], bad_len);
    if (bad_page) atomicAdd(&sums[1], bad_page);
    if (bad_list) atomicAdd(&sums[2], bad_list);
    if (first_bad != INT32_MAX) atomicMin(&first, first_bad);
    __syncthreads();
    if (tid < 3) a.counts[tid] = sums[tid];
    if (tid == 3) a.counts[3] = first == INT32_MAX ? -1 : first;
}

hipError_t launch_validate_paged(const ValidateArgs& a, hipStream_t st)
{
    hipLaunchKernelGGL(validate_paged_kernel, dim3(1), dim3(256), 0, st, a);
    return hipGetLastError();
}

// zero the arrival tickets of the fused split-KV entry point (a fill kernel, so that it can be captured in a graph)
__global__ __launch_bounds__(256) void clear_tickets_kernel(uint32_t* tickets, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) tickets[i] = 0u;
}

hipError_t launch_clear_tickets(uint32_t* tickets, int n, hipStream_t st)
{
    hipLaunchKernelGGL(clear_tickets_kernel, dim3((n + 255) / 256), dim3(256), 0, st, tickets, n);
    return hipGetLastError();
}

}  // namespace fck
