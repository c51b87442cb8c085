// A step's block tables go to the GPU as the rows and columns that the step uses: `rows` requests by the pages
// of the longest of them, out of a table as wide as the longest context the engine allows.  One strided copy
// from the pinned staging buffer, in the stream's order like the copy of the step's other arrays.  (The
// reference sends its packed metadata buffer whole each step: v3/crates/rvllm-metadata/src/layout.rs:19-78;
// its tables are as wide as the batch's longest context, rebuilt per step.)
#include "common.h"

extern "C" int rv_copy_rows_to_device(hipStream_t stream, void* dst, long long dst_pitch, const void* src,
                                      long long src_pitch, long long width_bytes, long long rows) {
  RV_CHECK(dst && src && rows >= 0 && width_bytes >= 0 && dst_pitch >= width_bytes && src_pitch >= width_bytes,
           "copy_rows: %lld rows of %lld bytes do not fit pitches %lld and %lld", rows, width_bytes, dst_pitch,
           src_pitch);
  if (rows == 0 || width_bytes == 0) return 0;
  const hipError_t err = hipMemcpy2DAsync(dst, (size_t)dst_pitch, src, (size_t)src_pitch, (size_t)width_bytes,
                                          (size_t)rows, hipMemcpyHostToDevice, stream);
  if (err != hipSuccess) return rv_fail("copy_rows: %s", hipGetErrorString(err));
  return 0;
}
