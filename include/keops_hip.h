/*
 * libkeops_hip - C ABI of the MI355X (gfx950) map-reduce backend.
 *
 * These entry points are what the reference's two FFI surfaces for its GPU path bind to:
 *   (1) the ctypes call  Compile(target_file, cu_code, use_half, use_fast_math, device_id,
 *       cuda_include_path)  of keopscore/keopscore/binders/nvrtc/nvrtc_jit.cpp:38-136
 *       (called from keopscore/keopscore/binders/nvrtc/Gpu_link_compile.py:78-91), and
 *   (2) the pybind11 class KeOps_module_{float,double}(device_id, nargs, target_file) with its
 *       __call__  (pykeops/pykeops/common/keops_io/pykeops_nvrtc.cpp:13-103), i.e.
 *       KeOps_module<TYPE>::launch_kernel of keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:328-643.
 *
 * Conventions: plain C types only; every pointer argument is borrowed for the duration of the
 * call; functions return 0 on success and a non-zero code on failure, with a human-readable
 * message available from keops_hip_last_error() (thread-local).  No exceptions cross the ABI.
 * A module must not be launched from two threads at once (same rule as the reference, whose
 * module owns a per-module argument buffer); distinct modules are independent.
 */
#ifndef KEOPS_HIP_H
#define KEOPS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Version of this ABI (bumped on any signature change). */
int keops_hip_abi_version(void);

/* sha256 of the embedded kernel templates and host code this library was built from; part of the
   key of the on-disk JIT cache (the reference hashes its own version into the tag,
   keopscore/keopscore/binders/LinkCompile.py:19-35). */
const char* keops_hip_templates_digest(void);

/* Number of visible HIP devices (0 when no GPU / no driver). */
int keops_hip_device_count(void);

/*
 * JIT-compile a kernel module with hiprtc and write it to target_file.
 * Replaces Compile() of nvrtc_jit.cpp:38-136.  hip_src is the generated plug-in (formula body +
 * geometry macros) that #includes one of the library's embedded kernel templates
 * ("keops_conv.h", ...).  The target architecture is taken from device_id when a device is
 * present, else from the environment variable KEOPS_HIP_ARCH, else "gfx950".
 * File format: [u64 code_size][code object][u64 meta_size][meta text]; the meta text is the
 * "//@keops key=value" lines of hip_src.  Returns 0 or the hiprtcResult.
 */
int keops_hip_compile(const char* target_file, const char* hip_src, int use_fast_math, int device_id);

/*
 * Load a compiled module on a device.  Replaces the KeOps_module<TYPE> constructor
 * (keops_nvrtc.cpp:354-380).  Returns an opaque handle, or NULL on error.
 */
void* keops_hip_module_create(int device_id, int nargs, const char* target_file);

/* Unload the module and free what it owns (keops_nvrtc.cpp:382-388). */
void keops_hip_module_destroy(void* module);

/*
 * Run one map-reduce.  Replaces KeOps_module<TYPE>::launch_kernel (keops_nvrtc.cpp:390-643);
 * arguments keep the reference's meaning and order:
 *   tagHostDevice     1: out, args and ranges[0..5] are device pointers.  0: they are host pointers
 *                     (load_args_FromHost / range_preprocess_from_host of the reference,
 *                     keopscore/keopscore/include/utils_pe.h:66-99, keops_nvrtc.cpp:250-325): the library copies
 *                     them into one pooled device allocation owned by the module, runs the same kernels, copies
 *                     out back and returns once it is in host memory (whatever `sync` says)
 *   dimY              total dimension of the reduced-index variables
 *   nx, ny            sizes M and N of the i and j axes (per batch)
 *   tagI              0: output indexed by i (reduce over j); 1: output indexed by j
 *   tagZero           1: the formula is identically zero: out is filled with zeros by a fill kernel on hip_stream and
 *                     nothing else runs.  A module is still required (it gives the element size); the engine
 *                     compiles none for a zero formula, so keops_amd/keops_io.py fills out itself and never
 *                     passes 1 here
 *   use_half          1: out and the arguments are arrays of IEEE half precision (device pointers, plain row-major
 *                     layout -- not the half2 interleaving that pykeops/pykeops/torch/half2_convert.py produces for
 *                     the CUDA kernels); the module must be compiled for float: the library converts the arguments
 *                     into a staging buffer owned by the module, computes in float32 and rounds the result to half
 *                     once (the reference computes in half2 arithmetic)
 *   tag1D2D           0: one pass over the reduced axis; 1: force the column-slab (2D) scheme
 *   dimred, dimout    accumulator and output dimensions per row
 *   block_size        upper bound for the workgroup size (0 = module default)
 *   use_chunk_mode    0 plain, 1 chunked inner reduction, 2 final chunks, 3 matrix-core K-nearest neighbours
 *                     (informative: the scheme is a property of the compiled module)
 *   indsi/j/p, dims*  argument indices and dimensions of the i, j and parameter variables
 *   ranges            7 pointers: ranges_i, slices_i, redranges_j, ranges_j, slices_j, redranges_i
 *                     (int64, on the data's device) and a HOST int64[6] with their row counts;
 *                     ranges[6][0] == -1 means "no ranges" (LoadKeOps.py:11-12,194-202).  The first launch of a
 *                     module with a given set of range tensors (same pointers and sizes) reads them back, checks
 *                     every index against its axis and fails with a message otherwise, as the reference reads
 *                     ranges_i back at every call (keops_nvrtc.cpp:195-197).  Later launches with the same tensors
 *                     build the workgroup table on the device from the tensors' current contents: no read-back,
 *                     no synchronisation, can be recorded in a HIP graph; indices that are out of bounds by then
 *                     are clamped and reported by keops_hip_ranges_status (KEOPS_HIP_DEVICE_RANGES=0: always the
 *                     first kind)
 *   shapeout          shape of out; out has prod(shapeout) elements
 *   args, argshapes   nargs device pointers; their shapes are concatenated in argshapes_flat,
 *                     argndims[k] entries each
 *   hip_stream        hipStream_t to launch on (NULL = default stream)
 *   sync              non-zero: wait for completion before returning (the reference always does)
 * Returns 0 or a hipError_t / negative library code.  KEOPS_HIP_NOT_CERTIFIED: a K-nearest-neighbour module for
 * vectors of more than 256 components ranks candidates found with reduced-precision products; when ties or
 * near-ties at the K-th distance keep it from proving that no reference was left out, it returns this code, `out`
 * is not valid and the caller runs the same call on a module compiled without the matrix-core schemes,
 * as keops_amd/keops_io.py does.  No counterpart in the reference, whose chunked kernels
 * (GpuReduc1D_chunks.py) accumulate in float32.
 */
#define KEOPS_HIP_NOT_CERTIFIED (-7)
int keops_hip_launch(void* module, int tagHostDevice, int64_t dimY, int64_t nx, int64_t ny, int tagI,
                     int tagZero, int use_half, int tag1D2D, int64_t dimred, int64_t block_size, int use_chunk_mode,
                     const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                     int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                     int64_t* const* ranges, const int64_t* shapeout, int nshapeout, void* out,
                     void* const* args, const int64_t* argshapes_flat, const int* argndims,
                     void* hip_stream, int sync);

/* Message describing the last failure on the calling thread ("" if none). */
const char* keops_hip_last_error(void);

/* Text of a "//@keops" metadata entry of a loaded module (NULL if absent); for diagnostics. */
const char* keops_hip_module_meta(void* module, const char* key);

/*
 * Time in milliseconds between two HIP events recorded on the launch stream around the main kernels of
 * the most recent keops_hip_launch on this module (the sweep over the pairs; pre-passes that prepare
 * operands and the final merge of slab partials lie outside), when timing has been enabled with
 * keops_hip_module_set_timing(module, 1); -1 if unavailable.  With timing on, a launch waits for its second event.
 * No counterpart in the reference (it only has commented-out clock() stamps,
 * keops_nvrtc.cpp:402-412); used by the benchmark's roofline measurement.
 */
void keops_hip_module_set_timing(void* module, int enabled);
double keops_hip_module_last_kernel_ms(void* module);

/*
 * keops_hip_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose launch_kernel allocates and
 * frees its tables inside every call (keops_nvrtc.cpp:468-481,632-640).  Same meaning of the arguments as
 * keops_hip_launch with tagHostDevice = 1, no ranges and no batch dimensions; the launch is asynchronous on
 * hip_stream.  Every workspace the kernels need (column-slab partial accumulators, the operand copies and
 * partials of the matrix-core chunked and final-product schemes) is taken from a static device buffer of
 * keops_hip_noalloc_scratch_bytes() = 128 MiB that each GPU holds from its first use until the process ends; the
 * call performs no hipMalloc / hipFree / hipHostMalloc and creates no events.  A launch whose workspace exceeds the
 * buffer, block-sparse or batched launches (they build device tables) and the K-nearest-neighbour schemes (they
 * read flags back through pinned memory) are refused with an error.  All calls on one GPU share the buffer:
 * calls that overlap on one GPU (two streams, two threads, or a captured graph replayed beside an eager call) race.
 */
int keops_hip_launch_noalloc(void* module, int64_t nx, int64_t ny, int tagI, int tag1D2D, int64_t dimred,
                             const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                             int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                             const int64_t* shapeout, int nshapeout, void* out, void* const* args,
                             const int64_t* argshapes_flat, const int* argndims, void* hip_stream);
size_t keops_hip_noalloc_scratch_bytes(void);

/*
 * Status of the module's block-sparse launches whose table was built on the device (see `ranges` above); waits for
 * the last launch.  Ranges are read back and validated on the host the first time a launch sees them; the key of
 * "the same ranges" is the identity of the six buffers (addresses and row counts), not their contents.  Later
 * launches build the table on the device, clamp every index to its axis and record what happened in two sticky
 * words: *status bit 0: an index of the ranges was out of bounds and has been clamped, bit 1: the row ranges overlap
 * so much that they need more workgroups than rows allow (the surplus was dropped).  Reading clears them; a
 * block-sparse launch that finds them set by an earlier launch fails with a message, so a clamped result never goes
 * unnoticed.  Host-pointer launches (tagHostDevice = 0) validate on the host at every call.  No counterpart in the
 * reference, which validates nothing (Sizes.h:12).
 */
int keops_hip_ranges_status(void* module, unsigned* status);

/*
 * Which of a module's two kernel families served its last launch; waits for that launch.  Two kinds of module
 * choose on the device, per launch, without host synchronisation: (1) Gaussian-type sums (meta key radial=1):
 * exponents from the matrix cores when the kernel is not too narrow for the cloud (block-sparse launches: for every
 * row range), the general-purpose kernel from exact differences otherwise; (2) K-nearest-neighbour modules with
 * knn_i8=1: the fixed-threshold filter on signed bytes when the quantisation slack is small against the search
 * radii, the bfloat16 filter otherwise (the returned neighbours are the same either way).  *taken: 1 the first of
 * the two ran, 0 the other one (or the module has one family only, or the launch was too small to try).
 * No counterpart in the reference.
 */
int keops_hip_path_status(void* module, unsigned* taken);

#ifdef __cplusplus
}
#endif
#endif /* KEOPS_HIP_H */
