/* C-ABI of libspnc_hip: batched joint log-likelihood inference of Sum-Product Networks on
 * AMD MI355X (gfx950).  Plain pointers and sizes only; every function returns 0 on success
 * and a non-zero code on failure, with the message available from spnc_hip_last_error().
 *
 * Each entry point names the interface of the reference SPN compiler (SPNC) it stands in for
 * when the compilation target is "HIP".
 */
#ifndef SPNC_HIP_H
#define SPNC_HIP_H

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define SPNC_HIP_API __attribute__((visibility("default")))
#else
#define SPNC_HIP_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque compiled kernel; the counterpart of spnc::Kernel (common/include/Kernel.h:29-126)
 * together with the runtime's cached Executable (runtime/src/Executable.cpp:41-133). */
typedef struct spnc_hip_kernel spnc_hip_kernel;

enum { SPNC_HIP_QUERY_JOINT = 1 };                      /* KernelQueryType, Kernel.h:20 */
enum { SPNC_HIP_TARGET_CPU = 1, SPNC_HIP_TARGET_CUDA = 2, SPNC_HIP_TARGET_HIP = 3 }; /* KernelTarget, Kernel.h:22 (+HIP) */
enum { SPNC_HIP_KERNEL_JIT = 1, SPNC_HIP_KERNEL_INTERPRETER = 2 };

/* The ten metadata fields of spnc::Kernel (Kernel.h:40-58) plus what the HIP target adds. */
typedef struct spnc_hip_info {
  char file_name[1024];      /* Kernel::fileName(): the serialized kernel on disk */
  char kernel_name[256];     /* Kernel::kernelName() */
  unsigned query_type;       /* Kernel::queryType() */
  unsigned target;           /* Kernel::target() == SPNC_HIP_TARGET_HIP */
  unsigned batch_size;       /* Kernel::batchSize() */
  unsigned num_features;     /* Kernel::numFeatures() */
  unsigned bytes_per_feature;/* Kernel::bytesPerFeature() */
  unsigned num_results;      /* Kernel::numResults() == 1 */
  unsigned bytes_per_result; /* Kernel::bytesPerResult() */
  char dtype[16];            /* Kernel::dataType(): "float32" or "float64" */
  /* HIP-target extras */
  unsigned kernel_kind;      /* SPNC_HIP_KERNEL_JIT or SPNC_HIP_KERNEL_INTERPRETER */
  unsigned input_alignment;  /* required alignment in bytes of device input pointers */
  unsigned num_nodes;        /* DAG nodes after dropping unreachable and merging identical ones */
  unsigned num_gaussian, num_categorical, num_histogram, num_product, num_sum;
  unsigned max_fan_in;
  uint64_t sum_terms;        /* sum over sum nodes of their child count */
  uint64_t product_adds;     /* sum over product nodes of (children - 1) */
  uint64_t flops_min;        /* algorithmic flops per sample, cheaper sum formulation per node */
  uint64_t trans_min;        /* of which transcendental */
  uint64_t flops_pairwise;   /* algorithmic flops per sample of the reference's pairwise trees */
  uint64_t trans_pairwise;
  uint64_t fused_min;        /* multiply-add pairs among flops_min that one fused instruction computes in log space
                                (Gaussian leaves and the product adds they feed): issue slots = flops_min - fused_min + 3 * trans_min */
  unsigned feature_is_float; /* 1: inputs are IEEE floats of bytes_per_feature bytes; 0: unsigned integers of that width (signed
                                integer arrays of the same width are read as unsigned, as the reference's index_cast / uitofp do) */
  unsigned support_marginal; /* the query was compiled with NaN-marginalisation */
  unsigned num_tasks;        /* kernels one execution launches: 1, or the tasks a graph was cut into by "maxTaskSize" */
  unsigned task_rows;        /* rows of intermediate values that pass between those tasks (each as long as the batch) */
} spnc_hip_info;

/* spn_compiler::isTargetSupported("HIP") (compiler/src/Driver.cpp:47-59): 1 if a gfx950 device
 * is visible to this process, else 0. Never fails. */
SPNC_HIP_API int spnc_hip_available(void);

/* spn_compiler::compileQuery(inputFile, options) (compiler/include/spnc.h:30, compiler/src/Driver.cpp:22-44).
 * query_path: Cap'n Proto stream file holding Header{query{joint}} of
 * xspn/xspn/serialization/binary/capnproto/spflow.capnp. keys/vals: n_opts string options
 * (must contain "target" = "HIP"). Needs no GPU: device code is produced here, loaded on first execute. */
SPNC_HIP_API int spnc_hip_compile(const char* query_path, const char* const* keys, const char* const* vals, size_t n_opts,
                     spnc_hip_kernel** out);

/* Accessors of spnc::Kernel (common/include/Kernel.h:60-104). */
SPNC_HIP_API int spnc_hip_kernel_info(const spnc_hip_kernel* k, spnc_hip_info* info);

/* spn_runtime::execute(kernel, num_elements, inputs, outputs) (runtime/include/spnc-runtime.h:36,
 * runtime/src/Executable.cpp:105-114): in = host buffer [n, num_features] row-major of the
 * compiled feature type, out = host buffer [n] of the result type. Blocks until out is written. */
SPNC_HIP_API int spnc_hip_execute(spnc_hip_kernel* k, size_t n, const void* in, void* out);

/* Device-resident variant of the same call: d_in/d_out are device pointers, the launch is
 * enqueued on `stream` (a hipStream_t, NULL for the default stream) and not waited for.
 * Replaces the host function the reference generates around its GPU kernel
 * (mlir/lib/Conversion/LoSPNtoGPU/GPUStructurePatterns.cpp:96-146) minus its copies. */
SPNC_HIP_API int spnc_hip_execute_device(spnc_hip_kernel* k, size_t n, const void* d_in, void* d_out, void* stream);

/* Allocation-free variant of spnc_hip_execute_device for interpreter kernels (compiled with "hip-kernel" =
 * "interpreter", or chosen for large graphs). It has no counterpart in the reference: it exists for callers that
 * cannot allocate device memory where they call it (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc). Same arguments and results as spnc_hip_execute_device; the library itself makes no hipMalloc,
 * hipFree, hipHostMalloc or hipHostFree call on this path (what the HIP runtime does inside a launch or a copy is
 * its own). Every device buffer the kernel needs besides d_in and d_out (instruction stream, leaf tables,
 * staged-feature descriptors, spilled value slots) lies in one fixed array of SPNC_HIP_STATIC_SCRATCH_BYTES inside
 * the library, one copy per GPU, held until the process ends. The first call with a kernel on a device, and the
 * first after another kernel used the array, copies the kernel's program into it on `stream` from pageable host
 * memory (make that call outside graph capture; the copy may block the host); later calls only launch. The launch
 * uses as many blocks as have room for their spilled slots in the array, so large programs run with a smaller grid
 * than spnc_hip_execute_device would give them, with identical results. A program whose stream, tables and one
 * block's spilled slots exceed the array, and a straight-line kernel (loading its code object allocates), are
 * refused with an error, and so is a call made with another device current than the kernel's first call saw. All
 * calls on one GPU share the array, from any thread or kernel handle: a call on another stream than the previous
 * call's waits for that call's kernel through an event (created when the array's address is resolved, i.e. on the
 * process's first call on that GPU), so calls on several streams run one after the other instead of racing. Calls on
 * a stream that is being captured into a graph are not ordered by the library: order such graphs' launches yourself. */
#define SPNC_HIP_STATIC_SCRATCH_BYTES (64u << 20)
SPNC_HIP_API int spnc_hip_execute_device_static(spnc_hip_kernel* k, size_t n, const void* d_in, void* d_out, void* stream);

/* Generated device source (JIT kernels) or program listing (interpreter), valid while k lives;
 * what the reference prints under "dump-ir". */
SPNC_HIP_API int spnc_hip_kernel_source(const spnc_hip_kernel* k, const char** text, size_t* len);

/* Re-creates a kernel from the file spnc_hip_info.file_name names; counterpart of constructing
 * spnc::Kernel from its metadata (python-interface/src/python-interface.cpp:22-23) and
 * Executable::initialize (runtime/src/Executable.cpp:116-133). */
SPNC_HIP_API int spnc_hip_load(const char* kernel_file, spnc_hip_kernel** out);

/* Releases device buffers, the loaded module and the handle (the kernel file stays on disk,
 * owned by the caller as in python-interface/spnc/gpu.py:212). */
SPNC_HIP_API void spnc_hip_destroy(spnc_hip_kernel* k);

/* Message of the last failure on the calling thread; "" if none. */
SPNC_HIP_API const char* spnc_hip_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* SPNC_HIP_H */
