// Entry points for callers that cannot allocate.
//
// rv_argmax_no_alloc has no counterpart in the reference.  It is for callers
// that may not call hipMalloc while they run: code under HIP graph capture,
// tight serving loops, harnesses that forbid allocation.  It computes what
// rv_argmax computes (the same two kernels: NaN skipped, equal maxima give the
// lowest id, a row of NaN gives id 0), but the partial results of the first
// stage go to a fixed array in device memory that the library itself holds,
// instead of a workspace the caller brings.
//
//   * The array holds RV_NO_ALLOC_MAX_ROWS x RV_NO_ALLOC_MAX_PARTS (value, id)
//     pairs: 512 KiB on every GPU the library is used on, until the process
//     ends.  rows above RV_NO_ALLOC_MAX_ROWS are refused with an error.
//   * The call allocates nothing and frees nothing, on the host's side of the
//     GPU or through any library; the caller passes the logits and the output.
//   * Every call on a GPU uses that GPU's one array, which keeps what the last
//     call left there.  A call reads only the slots that its own first stage
//     has written, so nothing needs clearing; but two calls that overlap on
//     one GPU (two streams, two threads) race for the array.  Calls on one
//     stream follow one another and are safe.
//   * The device that is current when the call is made must be the device of
//     the stream and of the pointers.
//   * The address of the array on a device is looked up once per device, which
//     may load the library's code onto that device: rv_no_alloc_init() does it
//     for the current device.  A caller that will call rv_argmax_no_alloc while
//     a stream is being captured, or from a place where nothing may be loaded,
//     calls rv_no_alloc_init() first, once per device, outside any capture.
//     Without it the first rv_argmax_no_alloc on a device does the same look-up
//     itself, and must then not be made under capture.
#pragma once

#include <hip/hip_runtime.h>

#define RV_NO_ALLOC_MAX_ROWS 256
#define RV_NO_ALLOC_MAX_PARTS 256

// Looks the array's address up for the current device (once; later calls return at once).  0 or an error code.
extern "C" int rv_no_alloc_init(void);

extern "C" int rv_argmax_no_alloc(hipStream_t stream, const float* logits, int rows, int vocab, long long row_stride,
                                  int* out);
