/*
 * cutt.h - tensor transpose plan API for AMD Instinct MI355X (gfx950).
 *
 * Drop-in for the plan API of cuTT: the four entry points, the handle type and
 * the result enum keep the names, argument order, argument meaning and enum
 * values of the reference header (reference src/cutt.h:31-41, 57-58, 76-77,
 * 88, 101); the only change in the signatures is hipStream_t where the
 * reference has cudaStream_t.  The symbols have C linkage, so the library can
 * be bound from C, C++ (source compatible with callers of the reference
 * header) and any FFI.
 *
 * Conventions (reference README.md:78-125):
 *   - dim[0] is the fastest running (contiguous) dimension of the input;
 *   - output dimension j is input dimension permutation[j], i.e. the output
 *     tensor has dimensions dim[permutation[0]], dim[permutation[1]], ...;
 *   - elements are opaque 4- or 8-byte values, moved bit-exactly;
 *   - transposes are out-of-place; idata and odata must not overlap;
 *   - dim and permutation are host arrays, read during the call only.
 */
#ifndef CUTT_H
#define CUTT_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same definition as in <hip/hip_runtime_api.h>; repeating a typedef is legal. */
typedef struct ihipStream_t* hipStream_t;

/* Handle that names a plan (reference src/cutt.h:31). */
typedef unsigned int cuttHandle;

/* Return values, same order and values as reference src/cutt.h:34-41. */
typedef enum cuttResult_t {
  CUTT_SUCCESS,            /* Success */
  CUTT_INVALID_PLAN,       /* Invalid plan handle */
  CUTT_INVALID_PARAMETER,  /* Invalid input parameter */
  CUTT_INVALID_DEVICE,     /* Execution tried on device different than where plan was created */
  CUTT_INTERNAL_ERROR,     /* Internal error */
  CUTT_UNDEFINED_ERROR     /* Undefined error */
} cuttResult;

/*
 * Create a plan; the method is chosen by the cost model.
 * Replaces reference cuttPlan (src/cutt.h:57-58, src/cutt.cpp:84-184).
 *
 *   handle            returned plan handle
 *   rank              rank of the tensor (>= 2)
 *   dim[rank]         dimensions, every one >= 2
 *   permutation[rank] a permutation of 0..rank-1
 *   sizeofType        element size in bytes, 4 or 8
 *   stream            HIP stream the plan executes on (0 = default stream)
 *
 * The plan is bound to the device that is current at the call.
 *
 * Sizes: up to 64 ranks and 2^46 elements.  One kernel launch addresses fewer than 2^32 elements;
 * a larger tensor (the reference's int volumes end at 2^31 - 1) is cut into pieces, and
 * cuttExecute issues one launch per piece on the plan's stream.  CUTT_INVALID_PARAMETER beyond
 * those sizes and for the shapes that have no such piece: those in which the rank that is
 * contiguous in the input lies 2^32 elements and more apart in the output, or the other way round -
 * (2, 70000, 70000) -> (70000, 70000, 2), 34 ranks of extent 2 reversed - and those in which a rank of
 * 2^31 entries and more has only tiny ranks beside it ((3, 2^31 - 1) transposed).
 */
cuttResult cuttPlan(cuttHandle* handle, int rank, int* dim, int* permutation,
                    size_t sizeofType, hipStream_t stream);

/*
 * Create a plan; every candidate is run on idata/odata, timed with HIP events,
 * and the fastest is kept.  Replaces reference cuttPlanMeasure
 * (src/cutt.h:76-77, src/cutt.cpp:186-284).
 *
 *   idata, odata      device buffers of product(dim)*sizeofType bytes.
 *                     The contents of odata are destroyed.
 *
 * Synchronises the device.
 */
cuttResult cuttPlanMeasure(cuttHandle* handle, int rank, int* dim, int* permutation,
                           size_t sizeofType, hipStream_t stream, void* idata, void* odata);

/*
 * Destroy a plan and free its device tables.  Replaces reference cuttDestroy
 * (src/cutt.h:88, src/cutt.cpp:286-294).  The caller makes sure that no
 * execution of the plan is still in flight.
 */
cuttResult cuttDestroy(cuttHandle handle);

/*
 * Execute a plan out-of-place, asynchronously on the plan's stream.  Replaces
 * reference cuttExecute (src/cutt.h:101, src/cutt.cpp:296-310).
 *
 *   idata, odata      device buffers of product(dim)*sizeofType bytes
 */
cuttResult cuttExecute(cuttHandle handle, void* idata, void* odata);

/*
 * Plan and execute in one call without allocating anything on the device.  No counterpart in the
 * reference; it is for callers that cannot allocate device memory where they transpose (tight
 * serving loops, harnesses that forbid hipMalloc): cuttPlan allocates a Packed / PackedSplit
 * plan's index tables with hipMalloc and copies them to the device, this call builds them with a
 * kernel on `stream` in static device memory of the library (1 MiB per GPU, held until the
 * process ends) and launches the same transpose kernel after it on `stream`.  The plan is the
 * one cuttPlan would choose; arguments and checks are those of cuttPlan and cuttExecute.
 *
 * Limits: tensors of 2^32 elements and more are refused (CUTT_INVALID_PARAMETER); a plan whose index
 * tables exceed the static memory is refused with
 * CUTT_INVALID_PARAMETER and a message on stderr (the tables of the plans this library builds
 * need at most 640 KiB).  Every call on one GPU uses the same static memory: calls on the same
 * stream are ordered and safe, calls whose work may overlap on the GPU (different streams, several
 * host threads) race and must be serialised by the caller.  The memory keeps the last call's
 * tables; every entry a call uses is rewritten by that call, nothing needs to start at zero.
 */
cuttResult cuttExecuteNoAlloc(int rank, int* dim, int* permutation, size_t sizeofType,
                              hipStream_t stream, void* idata, void* odata);

#ifdef __cplusplus
}
#endif

#endif /* CUTT_H */
