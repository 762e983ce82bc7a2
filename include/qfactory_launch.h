/*
 * C ABI of one compiled specialisation of the quantized-linear kernel.
 *
 * The JIT produces one shared object per (bits, group size, symmetric?, N, K, M, tiling).  Every
 * such object exports the entry points below; all problem and tiling parameters are constants
 * inside the object.  All pointers are device addresses owned by the caller, `stream` is a
 * hipStream_t, the call only enqueues work (no synchronisation), every element of `output` is
 * written exactly once (no pre-zeroing needed) and nothing of the caller's is retained after return.
 * The entry points are re-entrant with one exception, spelled out at launch_m_static below: an object whose
 * qf_describe names "KS=<blocks>" passes partial sums between its blocks through scratch memory it keeps per GPU, so
 * two launches of that one object must not run on one GPU at the same time (launches on one stream never do).
 *
 * Return code (written through the last argument): 0 launched, 1 the object's static
 * configuration is invalid (reason on stderr), 2 the HIP launch itself failed.
 *
 * A translation unit selects which of the two `launch` signatures it implements by defining
 * QF_LAUNCH_GROUPED or QF_LAUNCH_PLAIN before including this header; with neither defined only
 * the function-pointer types are declared (that is what a dlopen/dlsym or ctypes caller needs).
 */
#ifndef QFACTORY_LAUNCH_H
#define QFACTORY_LAUNCH_H

#ifdef __cplusplus
#define QF_RC_ARG int&
extern "C" {
#else
#define QF_RC_ARG int*
#endif

/*
 * Grouped-scale kernel: output (M,N) fp16 = activation (M,K) fp16 x dequant(weight, scale, zero)^T.
 *   weight (N, K*b/8) int8, scale (N, K/GS) fp16, zero (N, K/GS*b/8) int8 -- the packed layout of
 *   qfactory/convert.py:55-81; `zero` is ignored (may be any valid pointer) by symmetric objects.
 * Replaces the reference's generated
 *   extern "C" void launch(void* _activation, void* _weight, void* _output, void* _scale,
 *                          void* _zero, void* _stream, int& __return_code)
 * (emitted at qfactory/core/qfunc.py:133-152, bound through ctypes at qfactory/jit/runtime.py:37-49,
 *  implemented by gptq_gemv_impl, qfactory/include/gptq_gemv.h:156-205).  M is the object's constant.
 */
typedef void (*qf_launch_grouped_fn)(void* activation, void* weight, void* output, void* scale,
                                     void* zero, void* stream, int* return_code);

/*
 * Same computation for `m` activation rows (any m >= 1) instead of the object's constant M.
 * No counterpart in the reference, whose grouped kernel silently computes exactly its compile-time
 * M rows (qfactory/core/matmul.py:128 checks only activation.shape[0] == output.shape[0]).
 */
typedef void (*qf_launch_grouped_m_fn)(int m, void* activation, void* weight, void* output,
                                       void* scale, void* zero, void* stream, int* return_code);

/*
 * group_size == -1 kernel: output (m,N) fp16 = activation (m,K) fp16 x q^T with raw unsigned fields.
 * Replaces the reference's generated
 *   extern "C" void launch(int m, void* _activation, void* _weight, void* _output, void* _stream,
 *                          int& __return_code)
 * (emitted at qfactory/core/qfunc.py:263-316, implemented by gemv_impl, qfactory/include/gemv.h:96-135).
 */
typedef void (*qf_launch_plain_fn)(int m, void* activation, void* weight, void* output, void* stream,
                                   int* return_code);

/*
 * Grouped-scale kernel with the decoder layer's residual add and RMSNorm in front of its dot products (few rows;
 * fp16):  h = fp16(activation + delta)  (delta may be null),  a = fp16(fp16(h * rsqrt(mean(h^2) + eps)) * gamma),
 * output = a x dequant(weight)^T;  x_out (may be null; must not alias activation or delta) receives h.
 * gamma is the (K) fp16 RMSNorm weight.  Exported, besides launch / launch_m (which return 1: no norm operands),
 * by objects generated with the "add_rmsnorm" input prologue.  No counterpart in the reference, whose end-to-end
 * runs leave the step to vLLM's fused_add_rms_norm (third_party/vllm-qfactory.patch:205-214 calls the linear alone).
 */
typedef void (*qf_launch_grouped_norm_fn)(int m, void* activation, void* delta, void* gamma, void* x_out, float eps,
                                          void* weight, void* output, void* scale, void* zero, void* stream,
                                          int* return_code);

/*
 * launch_m without any allocation.  No counterpart in the reference; for callers that cannot allocate device memory:
 * code under HIP-graph capture from its first call on, tight serving loops, harnesses that forbid hipMalloc.
 * Exported only by objects whose kernel uses scratch memory beyond its inputs and outputs -- the A-stationary kernel
 * with long rows split over several blocks (qf_describe names "KS=<blocks>"), whose blocks exchange partial sums
 * through device memory.  launch / launch_m of such an object allocate that memory (hipMalloc, once
 * per device, at their first call there); launch_m_static uses a static device array of the object instead (at most
 * 8 MiB, one copy per GPU, held until the process ends) and calls no allocating routine.  Same arguments, same
 * result bits as launch_m.  At most 16 rows (32 for an object built for 17 .. 32); an object whose scratch memory would exceed the array returns 1 with a
 * message (call launch_m).  All calls on one GPU share the array: calls that overlap in time on one GPU race
 * (calls enqueued on one stream do not overlap).  The same holds for launch / launch_m of such an object among
 * themselves: they share the one buffer allocated per GPU (it is not the static array, so a launch_m and a
 * launch_m_static may overlap).  Layers of equal shape share one object; a caller that runs two of them on two
 * streams at once orders them with an event.  Every other object already allocates nothing in launch / launch_m
 * and keeps no state at all.
 */
typedef void (*qf_launch_grouped_m_static_fn)(int m, void* activation, void* weight, void* output,
                                              void* scale, void* zero, void* stream, int* return_code);

/* Static string naming the specialisation ("regime=gemv M=1 N=4096 K=4096 NBITS=4 ..."). */
typedef const char* (*qf_describe_fn)(void);

#if defined(QF_LAUNCH_GROUPED)
void launch(void* _activation, void* _weight, void* _output, void* _scale, void* _zero, void* _stream,
            QF_RC_ARG __return_code);
void launch_m(int m, void* _activation, void* _weight, void* _output, void* _scale, void* _zero,
              void* _stream, QF_RC_ARG __return_code);
const char* qf_describe(void);
#elif defined(QF_LAUNCH_PLAIN)
void launch(int m, void* _activation, void* _weight, void* _output, void* _stream, QF_RC_ARG __return_code);
const char* qf_describe(void);
#endif

#if defined(QF_LAUNCH_STATIC)
void launch_m_static(int m, void* _activation, void* _weight, void* _output, void* _scale, void* _zero,
                     void* _stream, QF_RC_ARG __return_code);
#endif

#if defined(QF_LAUNCH_NORM)
void launch_norm(int m, void* _activation, void* _delta, void* _gamma, void* _x_out, float eps, void* _weight,
                 void* _output, void* _scale, void* _zero, void* _stream, QF_RC_ARG __return_code);
#endif

#ifdef __cplusplus
}
#endif
#undef QF_RC_ARG

#endif /* QFACTORY_LAUNCH_H */
