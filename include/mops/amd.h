/* AMD-specific additions to the mops C ABI. None of these exist in
 * lab-cosmo/mops; callers that only use the reference's 61 symbols never
 * need them.
 *
 * Stream and synchronisation. The reference's device entry points launch on
 * the null stream and block until the device is idle
 * (e.g. mops/src/opsa/opsa.cu:85-87). That stays the default here. A caller
 * that manages its own HIP streams (PyTorch does) can instead name the
 * stream to launch on and turn the blocking wait off; both settings are per
 * calling thread.
 */
#ifndef MOPS_AMD_H
#define MOPS_AMD_H

#include <stdint.h>

#include "mops/exports.h"
#include "mops/tensor.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch all following mops_cuda_* calls of this thread on `hip_stream`
 * (a hipStream_t; NULL selects the null stream). Returns 0. */
MOPS_EXPORT int mops_amd_set_stream(void* hip_stream);

/* The stream set by mops_amd_set_stream on this thread (NULL by default). */
MOPS_EXPORT void* mops_amd_get_stream(void);

/* synchronous != 0 (default): every mops_cuda_* call waits for its kernels
 * before returning, as the reference does. synchronous == 0: calls return
 * once the work is enqueued; the caller orders later work on the same stream
 * or synchronises itself. Returns the previous setting. */
MOPS_EXPORT int mops_amd_set_synchronous(int synchronous);

/* Segment boundaries of a sorted index vector, on the device.
 *
 * `sorted_indices` holds n_input non-decreasing int32 values (device
 * memory). `first_occurrences` receives 2*n_output int32 values (device
 * memory): [v] is the position of the first element equal to v and
 * [n_output + v] one past the last; both are -1 for a value that does not
 * occur. Integer work, bit-exact. Replaces the reference's internal
 * calculate_first_occurences_cuda (mops/src/internal/cuda_first_occurences.cu:82-117),
 * which is what its scatter kernels use to find the rows of each output
 * segment; exposed here so the result can be checked on its own.
 * Returns 0 / 1 / 2 like every other entry point. */
MOPS_EXPORT int mops_amd_first_occurrences(
    const int32_t* sorted_indices, int64_t n_input, int64_t n_output, int32_t* first_occurrences
);

/* Device time of the main kernel of each operation (for benchmarks).
 *
 * mops_amd_kernel_timing(1) makes every following mops_cuda_* call of this
 * thread time its main kernel (the one that does the arithmetic; not the
 * small set-up kernels in front of it) with a pair of HIP events on the
 * stream it is launched on: attached to the launch itself where the kernel is
 * launched that way (sparse_accumulation_of_products), recorded just before
 * and after it otherwise. mops_amd_kernel_time waits for the recorded
 * events, stores the sum of the intervals in milliseconds and their number,
 * and forgets them. Calls captured into a HIP graph are not timed. The first
 * function returns the previous setting, the second 0 / 1 / 2. */
MOPS_EXPORT int mops_amd_kernel_timing(int enable);
MOPS_EXPORT int mops_amd_kernel_time(double* total_milliseconds, int64_t* launches);

/* Scatter indices that are not sorted.
 *
 * The device kernels of outer_product_scatter_add[_with_weights] and
 * sparse_accumulation_scatter_add_with_weights need their scatter index
 * (indices_output, indices_output_1) non-decreasing, as the device path of the
 * reference does (python/mops/tests/opsa.py:96); the reference's HOST path
 * accepts any order (mops/src/opsa/cpu.tpp:29). accept != 0 gives the calling
 * thread the host semantics on the device: each of these calls (forward, vjp,
 * vjp_vjp) first tests the index on the device and, when it is not sorted,
 * re-orders the edges by a stable sort, so that the result is the one the host
 * loops give. The test makes the call wait for the device once, so such calls
 * cannot be captured into a HIP graph. Default: off (or on when the
 * environment variable MOPS_AMD_ACCEPT_UNSORTED is set to something other
 * than 0). Returns the previous setting. */
MOPS_EXPORT int mops_amd_accept_unsorted_indices(int accept);

/* Scratch memory and HIP graphs.
 *
 * Some calls need temporary device memory (lists of the edges of every
 * sender, partial sums of very long segments). Each calling thread keeps one
 * block for it, which grows when a call needs more. Growing allocates, which
 * is not possible while the thread's stream is being captured into a graph: a
 * mops_cuda_* call that would have to grow the block during a capture fails
 * with status 1 and a message that says so. Before capturing, either make one
 * eager call with the largest shapes, or reserve the memory here.
 * mops_amd_reserve_scratch makes the calling thread's block at least `bytes`
 * large (0 / 1 / 2); mops_amd_scratch_capacity returns its present size.
 * A block that was used during a capture is never freed (a graph that was
 * captured may replay kernels that name it). */
MOPS_EXPORT int mops_amd_reserve_scratch(int64_t bytes);
MOPS_EXPORT int64_t mops_amd_scratch_capacity(void);

/* The entry point that allocates nothing.
 *
 * No counterpart in lab-cosmo/mops. It is for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc. Same arguments, checks, results (bit for bit) and
 * return convention as
 * mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32, but the
 * temporaries of its kernels (the dense coupling table and the list of every
 * sender's edges) live in an array of 4 MiB that is part of the library's
 * device code, one copy per GPU, held until the process ends; the call makes
 * no hipMalloc / hipFree and creates no stream or event (kernel timing,
 * mops_amd_kernel_timing, takes events from a pool that it fills on demand:
 * it is off inside this call, whatever the thread's setting). Shapes whose
 * sums are empty (no column, table entry, edge or node) give zero gradients,
 * as there. Limits, reported as status 1 with a message: A.shape[1],
 * W.shape[1], output.shape[1] at most 16; temporaries within 4 MiB (about
 * 7800 nodes); when grad_W is asked for together with grad_A or grad_B, at
 * most 48 edges per node on average and W.shape[1], output.shape[1] in the
 * same multiple of four; no grad_W at all for graphs so large and dense that
 * the edges are first sorted by sender; indices_output_1 sorted
 * (mops_amd_accept_unsorted_indices does not apply). With
 * MOPS_AMD_CHECK_INDICES=1 the indices are copied to the host and checked as
 * in the existing entry point, which waits for the stream and allocates host
 * memory: a debugging aid, not for a stream that is being captured. All calls
 * on one GPU share the array: calls that overlap on one GPU (two streams, two
 * threads) race; the caller serialises them. Nothing in the array needs to be
 * zero at entry. Runs on the calling thread's stream (mops_amd_set_stream);
 * with mops_amd_set_synchronous(0) a call can be captured into a HIP graph. */
MOPS_EXPORT int mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32(
    mops_tensor_2d_f32_t grad_A,
    mops_tensor_2d_f32_t grad_B,
    mops_tensor_3d_f32_t grad_W,
    mops_tensor_3d_f32_t grad_output,
    mops_tensor_2d_f32_t A,
    mops_tensor_2d_f32_t B,
    mops_tensor_1d_f32_t C,
    mops_tensor_3d_f32_t W,
    mops_tensor_1d_i32_t indices_A,
    mops_tensor_1d_i32_t indices_W_1,
    mops_tensor_1d_i32_t indices_W_2,
    mops_tensor_1d_i32_t indices_output_1,
    mops_tensor_1d_i32_t indices_output_2
);

#ifdef __cplusplus
}
#endif

#endif
