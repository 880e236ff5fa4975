// Device-wide stable segmented radix sort (descending) of whole rows: SampleTopK beyond the selection kernel's limits
// (sr_wide_rows_launch).  Equal keys keep their input order, which is ascending token index.
#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>

#include "sr_kernels.h"

hipError_t sr_segmented_sort_desc(void* tmp, size_t* tmp_bytes, const uint32_t* keys_in, uint32_t* keys_out,
                                  const int32_t* vals_in, int32_t* vals_out, int64_t n_items, int n_segments,
                                  const int32_t* seg_begin, const int32_t* seg_end, hipStream_t st)
{
    return hipcub::DeviceSegmentedRadixSort::SortPairsDescending(tmp, *tmp_bytes, keys_in, keys_out, vals_in, vals_out,
                                                                 (int)n_items, n_segments, seg_begin, seg_end, 0, 32, st);
}
