/* C ABI of libtts_hip.so: the MI355X execution backend behind triton-shared's
 * plugin surface.  Plain pointers and sizes only; no Python, torch or C++ types.
 *
 * Every entry point returns a tts_status.  On a non-zero status
 * tts_last_error() (thread-local) holds a message.  Strings returned through
 * `char **out` are malloc'd by the library and released with tts_free().
 *
 * Each declaration cites the reference interface it replaces (paths relative to
 * the triton-shared source tree).
 */
#ifndef TTS_HIP_H
#define TTS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tts_status {
  TTS_OK = 0,
  TTS_UNSUPPORTED = 1, /* the kernel is outside what this backend implements (NotImplementedError) */
  TTS_INVALID = 2,     /* malformed input or bad argument (ValueError / TypeError) */
  TTS_HIP_ERROR = 3    /* a HIP runtime call failed (RuntimeError) */
} tts_status;

/* One kernel argument, in the order of the tt.func signature (constexpr
 * parameters are not arguments).  Replaces the per-argument C parameters of the
 * generated kernel symbol, backend/driver.py:96-100,109-114: a pointer was
 * "int64_t rank, void *descriptor", a scalar was passed by value. */
typedef enum tts_arg_kind { TTS_ARG_PTR = 0, TTS_ARG_INT = 1, TTS_ARG_FLOAT = 2 } tts_arg_kind;
typedef struct tts_arg {
  int32_t kind; /* tts_arg_kind */
  int32_t reserved;
  union {
    void *ptr;  /* device pointer (may be NULL if the kernel never dereferences it) */
    int64_t i;  /* i1/i8/i16/i32/i64 and unsigned scalars, sign- or zero-extended */
    double f;   /* fp32/fp64 scalars */
  } v;
} tts_arg;

typedef struct tts_plan tts_plan;

/* TTIR text -> structured program text.
 * Replaces the `triton-shared-opt --triton-to-linalg-experimental` subprocess of
 * backend/compiler.py:48-67 (pipeline: lib/Conversion/TritonToLinalgExperimental/
 * TritonToLinalgExperimentalPass.cpp:52-88). */
tts_status tts_ttir_to_structured(const char *ttir_text, char **out);

/* Structured program text -> launch plan bytes (kernel family + bindings).
 * Replaces _ttsharedir_to_llir + _llir_to_bin, backend/compiler.py:75-175.
 * *out_name receives the kernel name (metadata["name"], compiler.py:133-136). */
tts_status tts_structured_to_plan(const char *structured_text, char **out_plan, size_t *out_len, char **out_name);

void tts_free(void *p);
const char *tts_last_error(void);

/* Plan bytes -> handle.  Replaces CPUUtils.load_binary, backend/driver.py:409-417
 * (there the "function" is the object file itself). */
tts_status tts_plan_load(const char *plan_bytes, size_t len, tts_plan **out);
void tts_plan_destroy(tts_plan *plan);
const char *tts_plan_kernel_name(const tts_plan *plan);
const char *tts_plan_family(const tts_plan *plan);   /* map1d, row_softmax, layernorm_fwd, gemm, gemm_w8a16 */
const char *tts_plan_signature(const tts_plan *plan); /* normalised op listing the family was recognised from */
int tts_plan_num_args(const tts_plan *plan);
/* kind of argument i: TTS_ARG_PTR / TTS_ARG_INT / TTS_ARG_FLOAT */
int tts_plan_arg_kind(const tts_plan *plan, int i);

/* Resolves the plan's bindings for one launch configuration without touching
 * the GPU and describes the kernel launch that tts_launch would issue, as
 * "key=value" lines.  Used by host-side tests; no counterpart in the reference. */
tts_status tts_plan_describe_launch(tts_plan *plan, int grid_x, int grid_y, int grid_z, const tts_arg *args,
                                    int num_args, char **out);

/* Enqueues the whole grid on `stream` (a hipStream_t; NULL = the null stream)
 * and returns without waiting.  Replaces _launch, backend/driver.py:116-133 (the
 * serial x/y/z loop over programs) together with the compiled kernel it calls.
 * A grid with zero volume is a no-op (driver.py:117). */
tts_status tts_launch(tts_plan *plan, int grid_x, int grid_y, int grid_z, void *stream, const tts_arg *args,
                      int num_args);

/* tts_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as tts_launch, but
 * the call never allocates or frees device memory and never compiles: the split-K partial tiles and arrival counters
 * of the int8-weight product, and the partial sums of a matrix product that runs in K slices, live in a static device
 * array (8 MiB + 4096 counters per GPU, held until the process ends; its address is looked up with
 * hipGetSymbolAddress at the first call on each device).  An int8-weight launch whose partial tiles exceed that, or
 * a launch that would need a run-time compiled kernel or a device-side table that no earlier tts_launch of the plan
 * has created yet, returns TTS_UNSUPPORTED with the reason; a matrix product runs in as many slices as fit there, or
 * without slices.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (two streams, two threads) race on it. */
tts_status tts_launch_noalloc(tts_plan *plan, int grid_x, int grid_y, int grid_z, void *stream, const tts_arg *args,
                              int num_args);

/* Name of the device kernel the last tts_launch on this plan used (for profiles). */
const char *tts_plan_last_kernel(const tts_plan *plan);

#ifdef __cplusplus
}
#endif
#endif /* TTS_HIP_H */
