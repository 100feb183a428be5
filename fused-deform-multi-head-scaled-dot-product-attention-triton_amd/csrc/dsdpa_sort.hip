// Ordering of the cell lists for the deterministic backward: every list (the samples of one bilinear
// cell of one (batch, key view)) sorted by sample id, so that the dk/dv kernel adds them up in the same
// order on every run. The counting sort that builds the lists places the samples of a cell in whatever
// order its atomics resolve; the ids inside a cell are distinct, so sorting them fixes the order.
// A plain segmented key sort: rocPRIM's device routine (no allocation: it works in the caller's workspace).
#include <cstring>

#include <hip/hip_runtime.h>
#include <rocprim/device/device_segmented_radix_sort.hpp>

#include "dsdpa_host.h"

namespace dsdpa {

size_t sort_temp_bytes(size_t n, size_t segments)
{
    size_t bytes = 0;
    hipError_t e = rocprim::segmented_radix_sort_keys(nullptr, bytes, (const unsigned *)nullptr, (unsigned *)nullptr,
                                                      (unsigned)n, (unsigned)segments, (const unsigned *)nullptr,
                                                      (const unsigned *)nullptr, 0u, 32u, (hipStream_t)0);
    if (e != hipSuccess) return 0;
    return bytes < 256 ? 256 : bytes;
}

int sort_cell_lists(void *temp, size_t temp_bytes, const unsigned *ids_in, unsigned *ids_out, size_t n,
                    size_t segments, const unsigned *seg_begin, const unsigned *seg_end, unsigned id_bits,
                    hipStream_t st)
{
    hipError_t e = rocprim::segmented_radix_sort_keys(temp, temp_bytes, ids_in, ids_out, (unsigned)n,
                                                      (unsigned)segments, seg_begin, seg_end, 0u, id_bits, st);
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return DSDPA_ERR_HIP;
    }
    return DSDPA_OK;
}

}  // namespace dsdpa
