/*
 * Thin C-ABI HIP runtime layer: what the host code of the tensor library calls
 * where the reference called EasyCL (device discovery, buffers, the in-order
 * queue, the runtime kernel cache and the timers).  Reference call sites this
 * replaces: `EasyCL::createForIndexedGpu` / `cl->wrap` / `CLWrapper::copyTo*` /
 * `cl->kernelExists|getKernel` / `TemplatedKernel::buildKernel` /
 * `CLKernel::run` / `cl->finish` / `StatefulTimer::*`
 * (src/lib/THClGeneral.cpp:134-165, src/lib/THClStorage.cpp:112-140,
 *  src/lib/THClApply.cpp:87-141, src/lib/THClKernels.cpp:156-176).
 *
 * One context per device, one in-order stream per context.  All functions
 * return 0 on success or a negative code; thcl_rt_error() gives the message.
 */
#ifndef THCL_RT_H
#define THCL_RT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility: what is declared here is what it exports */
#pragma GCC visibility push(default)

typedef struct thcl_rt thcl_rt;
typedef struct thcl_rt_kernel thcl_rt_kernel;

typedef struct thcl_rt_props {
  char name[128];
  char arch[64];
  int compute_units;
  int wavefront;
  int max_threads_per_block;
  int clock_khz;
  int lds_bytes_per_block;
  size_t total_mem;
} thcl_rt_props;

int thcl_rt_device_count(void);
/* lazily creates the context (stream + scratch) of `device`; NULL on failure */
thcl_rt *thcl_rt_get(int device);
void thcl_rt_release_all(void);
const thcl_rt_props *thcl_rt_get_props(thcl_rt *rt);
const char *thcl_rt_error(void);

/* buffers */
/* Released blocks are kept and handed out again (safe because each context has
 * one in-order stream); at most half the device's memory, or THCL_ALLOC_CACHE_MB
 * megabytes (0: no caching), stays cached, and the cache is emptied when the
 * driver runs out of memory. */
void *thcl_rt_malloc(thcl_rt *rt, size_t bytes);
int thcl_rt_free(thcl_rt *rt, void *dptr);
int thcl_rt_empty_cache(thcl_rt *rt);
void thcl_rt_memory_stats(thcl_rt *rt, size_t *live_bytes, size_t *cached_bytes, unsigned long long *device_mallocs,
                          unsigned long long *cache_hits);
int thcl_rt_memcpy_h2d(thcl_rt *rt, void *dst, const void *src, size_t bytes); /* returns when `src` may be reused;
                                                                                 * the stream sees the bytes in order */
int thcl_rt_memcpy_d2h(thcl_rt *rt, void *dst, const void *src, size_t bytes); /* returns when done */
/* `count` dense host elements of another type to or from device floats, converted by C casts on the way
 * (to_device != 0: host -> device).  Returns when done. */
enum { THCL_RT_U8 = 0, THCL_RT_I8 = 1, THCL_RT_I16 = 2, THCL_RT_I32 = 3, THCL_RT_I64 = 4, THCL_RT_F64 = 5 };
int thcl_rt_copy_converted(thcl_rt *rt, void *dev, void *host, size_t count, int kind, int to_device);
int thcl_rt_memcpy_d2d(thcl_rt *rt, void *dst, const void *src, size_t bytes); /* queued            */

/* queue */
void *thcl_rt_stream(thcl_rt *rt); /* hipStream_t */
int thcl_rt_sync(thcl_rt *rt);

/* per-device scratch block (partials, tickets), zero-initialised once */
void *thcl_rt_scratch(thcl_rt *rt, size_t *bytes);
/* a device buffer of at least `bytes` that lives until a larger one is asked
 * for; work queued on the stream keeps using it in order */
void *thcl_rt_workspace(thcl_rt *rt, size_t bytes);
/* pinned host words for handing scalars back */
float *thcl_rt_host_word(thcl_rt *rt);
/* the same words at the address kernels use: a kernel may leave a scalar there
 * directly, and the host reads it after thcl_rt_sync (no copy in between) */
float *thcl_rt_host_word_device(thcl_rt *rt);

/* A pinned word, at the address kernels use, that a kernel sets to non-zero when the host must hear
 * about something: 1 = an index outside its range (that entry moved nothing), 2 = a wait inside a
 * single-pass scan ran out because its blocks did not run at the same time (that scan's result is
 * not valid).  thcl_rt_sync and thcl_rt_memcpy_d2h look at it after they have waited: if it is set
 * they clear it and return -3 with a message. */
unsigned *thcl_rt_fault_word_device(thcl_rt *rt);
/* The same look without a wait, for a caller that has just waited for the stream by other means (its own event, a
 * copy through another library): 0, or -3 with the message after clearing the word. */
int thcl_rt_check_fault(thcl_rt *rt);

/* A scalar handed to the host without waiting for the stream's completion signal: a kernel that is given
 * thcl_rt_tagged_word_device() and a tag from thcl_rt_next_tag() writes {value, tag} there in one 8-byte store when
 * it has the value; thcl_rt_await_tagged() polls the pair for up to 2 ms and then falls back to
 * thcl_rt_sync().  Returns what thcl_rt_sync would (also -3 when the fault word is set).  Work queued behind the
 * kernel is unaffected: the stream stays in order.  The reference reads such scalars back with a blocking copy
 * (src/lib/THClTensorMath.cpp:346-368). */
float *thcl_rt_tagged_word_device(thcl_rt *rt);
/* Page-locked room behind those words for a small tensor on its way to the host: a kernel copies it there
 * (thcl_rt_mailbox_device), then stores the tagged pair; the host awaits the tag and reads thcl_rt_mailbox_host
 * (`floats` receives its size).  One copy at a time: the caller reads the mailbox before anything else uses it. */
float *thcl_rt_mailbox_device(thcl_rt *rt);
const float *thcl_rt_mailbox_host(thcl_rt *rt, size_t *floats);
unsigned thcl_rt_next_tag(thcl_rt *rt);
int thcl_rt_await_tagged(thcl_rt *rt, unsigned tag, float *value);

/* Page-locked host memory for callers that stage their own transfers: copies between a
 * tensor and such a buffer run at the link's rate (57 GB/s measured on MI355X; ordinary memory,
 * which the runtime moves through page-locked buffers of its own, gets 41-52).  The reference keeps its host mirrors
 * in ordinary memory (src/lib/THClStorage.cpp:112-140); this has no counterpart there. */
void *thcl_rt_host_alloc(size_t bytes);
int thcl_rt_host_free(void *ptr);

/* Runtime-compiled kernels (hipRTC), cached per context by `key`.  `source`
 * is complete HIP source; `entry` the extern "C" kernel name.  On a compile
 * error returns NULL and thcl_rt_error() holds the compiler log.  With the
 * environment variable THCL_KERNEL_CACHE_DIR set, compiled code objects are
 * also kept in that directory and loaded from it by later processes. */
thcl_rt_kernel *thcl_rt_kernel_get(thcl_rt *rt, const char *key, const char *source, const char *entry);
int thcl_rt_kernel_cached(thcl_rt *rt, const char *key);
int thcl_rt_launch(thcl_rt *rt, thcl_rt_kernel *k, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                   unsigned by, unsigned bz, unsigned lds_bytes, void *params, size_t params_bytes);
/* compile only (no device needed): returns 0 and the code-object size */
int thcl_rt_compile_check(const char *source, const char *arch, size_t *code_bytes);

/* event timers on the context's stream */
typedef struct thcl_rt_timer thcl_rt_timer;
thcl_rt_timer *thcl_rt_timer_new(thcl_rt *rt);
int thcl_rt_timer_start(thcl_rt_timer *t);
int thcl_rt_timer_stop(thcl_rt_timer *t);
float thcl_rt_timer_ms(thcl_rt_timer *t); /* waits for the stop event */
void thcl_rt_timer_free(thcl_rt_timer *t);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
