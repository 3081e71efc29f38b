/*
 * C ABI of the acrotensor "HIP" backend (libacrotensor_hip.so).
 *
 * The reference has no foreign-function interface: its boundary is the C++ classes acro::TensorEngine,
 * acro::Tensor, acro::SliceTensor, acro::IndexMapping (see the C++ headers next to this file, which keep that
 * API).  This header flattens exactly that boundary into extern "C" entry points with plain pointers and sizes
 * so that other languages can bind it; each entry point names the reference interface it stands for.
 *
 * Conventions: every function that can fail returns 0 on success and a non-zero code on failure (the C++
 * exception the reference would throw, util/Error.hpp:15-23, is caught at the boundary); acro_last_error()
 * then returns its message for the calling thread.  Handles are opaque.  All tensors are dense row-major fp64,
 * extents and indices are int.  Device work is asynchronous on one library-owned stream; the *_move_from_gpu
 * calls and acro_hip_synchronize() are the synchronisation points.
 */
#ifndef ACROTENSOR_HIP_H
#define ACROTENSOR_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct acro_engine acro_engine;
typedef struct acro_tensor acro_tensor;
typedef struct acro_index_mapping acro_index_mapping;

/* Message of the last failure on this thread ("" if none). */
const char *acro_last_error(void);
/* 1 when a HIP device is usable (reference: isCudaReady(), util/CudaUtil.hpp:175-184). */
int acro_hip_is_ready(void);
/* Block until all work issued by the library has finished. */
int acro_hip_synchronize(void);
/* Adopt an externally created hipStream_t (NULL: back to the library's own stream).  Stands in for the
 * reference's setCudaContext(), util/CudaUtil.hpp:93-98.  Work queued before the switch is ordered ahead of work
 * queued after it (an event on the outgoing stream that the incoming one waits for; the host does not wait).  An
 * adopted stream must stay alive until the library has been switched away from it: if the hand-over fails because
 * it is gone, the switch is still made and the call reports the failure (no ordering across that switch). */
int acro_hip_set_stream(void *hip_stream);
void *acro_hip_get_stream(void);

/* Timing on the library's stream with HIP events (measurement support; no reference counterpart). */
int acro_hip_event_create(void **event);
int acro_hip_event_record(void *event);
int acro_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for stop */
int acro_hip_event_destroy(void *event);

/* Recorded launch sequences (hipGraph): between begin_capture and end_capture every kernel the library would launch
 * on its stream is recorded instead of executed; acro_hip_graph_launch then enqueues the whole sequence with one
 * call, in stream order with everything else.  While recording, anything that needs the host fails (allocation,
 * host <-> device copies, synchronisation): tensors must be resident and the sequence must have run once before.
 * No counterpart in the reference, which launches kernel by kernel on the null stream (exec/CudaExecutor.cpp:70-101). */
typedef struct acro_hip_graph acro_hip_graph;
int acro_hip_graph_begin_capture(void);
int acro_hip_graph_end_capture(acro_hip_graph **out);  /* also ends a recording in which a call failed */
int acro_hip_graph_abort_capture(void);
int acro_hip_graph_launch(acro_hip_graph *g);
int acro_hip_graph_destroy(acro_hip_graph *g);

/* ---- acro::Tensor (tensor/Tensor.hpp:15-126) and acro::SliceTensor (tensor/SliceTensor.hpp:14-58) ---- */
/* hdata / ddata may be NULL (library-owned host buffer / no device mirror yet); ongpu marks the device copy
 * as the current one (Tensor::Init rules, tensor/Tensor.cpp:166-202). */
int acro_tensor_create(int rank, const int *dims, double *hdata, double *ddata, int ongpu, acro_tensor **out);
/* View of parent at the given leading indices (SliceTensor::SliceInit, tensor/SliceTensor.cpp:142-168).
 * The parent must outlive the slice. */
int acro_tensor_create_slice(acro_tensor *parent, int num_indices, const int *indices, acro_tensor **out);
int acro_tensor_destroy(acro_tensor *t);
int acro_tensor_rank(const acro_tensor *t);
long long acro_tensor_size(const acro_tensor *t);      /* entries; may exceed 2^31 */
int acro_tensor_dim(const acro_tensor *t, int d);
long long acro_tensor_stride(const acro_tensor *t, int d);
double *acro_tensor_data(const acro_tensor *t);        /* host buffer   (Tensor::GetData) */
double *acro_tensor_device_data(const acro_tensor *t); /* device mirror (Tensor::GetDeviceData), may be NULL */
int acro_tensor_reshape(acro_tensor *t, int rank, const int *dims);
int acro_tensor_retarget(acro_tensor *t, double *hdata, double *ddata);
int acro_tensor_map_to_gpu(acro_tensor *t);
int acro_tensor_move_to_gpu(acro_tensor *t);
int acro_tensor_switch_to_gpu(acro_tensor *t);
int acro_tensor_unmap_from_gpu(acro_tensor *t);
int acro_tensor_move_from_gpu(acro_tensor *t);
int acro_tensor_switch_from_gpu(acro_tensor *t);
int acro_tensor_is_mapped_to_gpu(const acro_tensor *t);
int acro_tensor_is_on_gpu(const acro_tensor *t);
int acro_tensor_set(acro_tensor *t, double value);   /* Tensor::Set,  tensor/Tensor.cpp:330-347 */
int acro_tensor_mult(acro_tensor *t, double factor); /* Tensor::Mult, tensor/Tensor.cpp:350-367 */
/* Extension without reference counterpart: a transient tensor is scratch of a fused multi-kernel launch; its
 * contents in device memory are unspecified after the launch (the store may be skipped). */
int acro_tensor_set_transient(acro_tensor *t, int transient);
/* Extension without reference counterpart (the reference allocates host buffers with new[], tensor/Tensor.cpp:196):
 * host buffers that the library allocates for tensors created from now on are page-locked, so that host <-> device
 * moves run at the rate of the host link.  Needs a HIP device. */
int acro_tensor_set_pinned_host_allocation(int pinned);

/* ---- acro::IndexMapping (tensor/IndexMapping.hpp:13-45) ---- */
int acro_index_mapping_create(int domain_size, int range_size, acro_index_mapping **out);
int acro_index_mapping_destroy(acro_index_mapping *m);
int *acro_index_mapping_data(acro_index_mapping *m); /* range_size ints, entry i = domain index of range entry i */
int acro_index_mapping_compute_inverse(acro_index_mapping *m);
int *acro_index_mapping_inverse_data(acro_index_mapping *m);    /* NULL before the inverse is computed */
int *acro_index_mapping_inverse_offsets(acro_index_mapping *m); /* domain_size+1 ints, NULL likewise */

/* ---- acro::TensorEngine (kernel/TensorEngine.hpp:26-114) ---- */
/* exec_type: "HIP" (the policy this library provides). */
int acro_engine_create(const char *exec_type, acro_engine **out);
int acro_engine_destroy(acro_engine *e);
int acro_engine_set_executor_type(acro_engine *e, const char *exec_type);
/* TensorEngine::operator()(kernel_str, out, inputs)  (kernel/TensorEngine.cpp:290-315) */
int acro_engine_contract(acro_engine *e, const char *kernel, acro_tensor *out, acro_tensor *const *inputs,
                         int num_inputs);
/* The same operation as acro_engine_contract for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc); no counterpart in the reference, whose launches never allocate
 * because its kernels have no scratch memory (exec/CudaExecutor.cpp:70-101).  This call allocates no device or
 * page-locked memory and loads no code object: every tensor must already be resident on the device, and the same
 * kernel string on tensors of the same extents must have run once through acro_engine_contract on that device (which
 * compiles and loads the kernel, and looks up the device address of the scratch array below: the first look-up on a
 * device may load code and allocate, so it is never done here); otherwise the call fails with a message saying so.  Kernels that need scratch memory beyond
 * their operands (split contractions such as "S_i_j = A_n_i_j B_n": per-workgroup partial sums) take it from one
 * array of ACRO_NO_ALLOC_SCRATCH_BYTES that the library holds on every device it runs on until the process ends; a
 * kernel that needs more is refused with a message.  All calls on a device share that array, which keeps the last
 * call's contents (the part a call uses is cleared first, on the stream): calls that overlap on one device, from
 * several threads or on several streams, race.  Results are bit-identical to acro_engine_contract's.  Not available
 * between acro_engine_begin_multi_kernel_launch and acro_engine_end_multi_kernel_launch (there a call is only
 * recorded, and the launch at the end is an ordinary one). */
#define ACRO_NO_ALLOC_SCRATCH_BYTES (256u * 1024u)
int acro_engine_contract_no_alloc(acro_engine *e, const char *kernel, acro_tensor *out, acro_tensor *const *inputs,
                                  int num_inputs);
/* Between begin and end, acro_engine_batch_matrix_inverse / _det / _inv_det are recorded as well and run at end, in
 * program order with the recorded kernels; an operation whose result a later recorded kernel reads is fused into the
 * launch (the reference runs these operations at the call, kernel/TensorEngine.cpp:627-671).  The same for
 * acro_engine_flat_indexed_scatter: with a transient result that only later recorded kernels read, those kernels read the
 * source through the map and the result is never written. */
int acro_engine_begin_multi_kernel_launch(acro_engine *e); /* kernel/TensorEngine.cpp:318-325 */
int acro_engine_end_multi_kernel_launch(acro_engine *e);   /* kernel/TensorEngine.cpp:328-336 */
/* TensorEngine::GetImplementation: copies the generated HIP source (NUL terminated, truncated to buflen) and
 * reports the full length in *needed.  Works without a device. */
int acro_engine_get_implementation(acro_engine *e, const char *kernel, acro_tensor *out,
                                   acro_tensor *const *inputs, int num_inputs, char *buf, size_t buflen,
                                   size_t *needed);
/* Ends a capture started by acro_engine_begin_multi_kernel_launch WITHOUT executing it and returns the source of
 * the fused kernel that the launch would have used.  Works without a device. */
int acro_engine_end_multi_kernel_get_implementation(acro_engine *e, char *buf, size_t buflen, size_t *needed);
/* Source of the kernel used by the most recent launch (also for multi-kernel launches). */
int acro_engine_get_last_implementation(acro_engine *e, char *buf, size_t buflen, size_t *needed);
int acro_engine_clear(acro_engine *e);
/* The five non-contraction operations (kernel/TensorEngine.cpp:627-714, ops/NonContractionOps.hpp:17-32) */
int acro_engine_batch_matrix_inverse(acro_engine *e, acro_tensor *Ainv, acro_tensor *A);
int acro_engine_batch_matrix_det(acro_engine *e, acro_tensor *Adet, acro_tensor *A);
int acro_engine_batch_matrix_inv_det(acro_engine *e, acro_tensor *Ainv, acro_tensor *Adet, acro_tensor *A);
int acro_engine_flat_indexed_scatter(acro_engine *e, acro_tensor *Aout, acro_tensor *Ain, acro_index_mapping *M);
int acro_engine_flat_indexed_sum_gather(acro_engine *e, acro_tensor *Aout, acro_tensor *Ain,
                                        acro_index_mapping *M);

/* ---- runtime compiler, host only (stands for CudaKernel::GenerateFunction, util/CudaUtil.cpp:43-84) ---- */
/* Compiles HIP C++ source for gfx950 with the options the library uses for generated kernels; needs no device.
 * Returns 0 and the code-object size in *code_size, or non-zero with the compiler log in acro_last_error(). */
int acro_hip_compile(const char *module_name, const char *source, size_t *code_size);
/* Compiles the same way and reports the private (scratch) memory per work item, in bytes, that the code object
 * declares for the kernel `function`: non-zero means register spills or arrays in private memory.  This is the figure
 * the library checks for every generated matrix-core kernel before it will launch it (such a kernel is compiled again
 * with its register-relief switch, and replaced by a schedule without the matrix cores if that does not help).
 * Diagnostics; the reference has no counterpart (NVRTC output is launched as it comes, util/CudaUtil.cpp:43-84). */
int acro_hip_compile_private_bytes(const char *module_name, const char *source, const char *function, int *bytes);

/* ---- kernel IR introspection, host only (kernel/TensorKernel.hpp, DimensionedKernel.hpp,
 *      DimensionedMultiKernel.hpp) ---- */
/* Parses num_kernels kernel strings and binds them to shapes.  For kernel k its tensors are listed output first,
 * then inputs: ranks[] holds one rank per tensor over all kernels, dims[] all extents back to back.  Writes a
 * JSON description (name strings, index lists, loop order, extents, sizes, unique variables) to buf. */
int acro_describe_kernels(int num_kernels, const char *const *kernels, const int *ranks, const int *dims,
                          char *buf, size_t buflen, size_t *needed);

#ifdef __cplusplus
}
#endif

#endif /* ACROTENSOR_HIP_H */
