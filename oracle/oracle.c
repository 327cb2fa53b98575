/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's CPU collective path for one rank's share
 * of reduce_scatter_tensor, all_gather_into_tensor and the compile_op copies.
 * Only tests, the smoke check and the cpu_baseline leg of the benchmark may
 * load this file's library.  The shipped path never calls it.
 *
 * Every function names the reference lines it follows.  What pins each one
 * (known answers, closed forms, brute force) is listed beside it:
 *
 *   orc_reduce      pinned: reference tests' known answers
 *                   (tests/test_processgroup.py:51-79 SUM of rank+1 = P(P+1)/2,
 *                   tests/test_stress.py:235-280 ragged sizes), the fp32
 *                   order witness [1e8,1,-1e8,1] -> 1, the bf16 witness
 *                   [1,2^-8,2^-8] -> 1+2^-7, signed-zero/NaN min/max cases,
 *                   and an independent torch-CPU element-wise fold.
 *   orc_gather      pinned: reference tests' known answers
 *                   (tests/test_processgroup.py:21-48, :82-109, :112-146) and
 *                   numpy slicing on small shapes.
 *   orc_copy_box    pinned: numpy basic slicing on small shapes (brute force).
 *   orc_cpu_reduce_scatter_ranks  timing harness only; its result is checked
 *                   against orc_reduce.
 *
 * No function here is left unpinned.  What the reference's OWN tests do not
 * cover -- and what is therefore pinned by the closed forms and torch
 * witnesses above only -- is: 16-bit floats, MIN/MAX/AVG/PREMUL_SUM, more than
 * eight sources, and strided (non-contiguous-slice) copies.
 *
 * dtype codes are torch ScalarType numbers and op codes are c10d RedOpType
 * numbers, as on the reference's API (api/moodist_api.h:30-55).
 */
#define _GNU_SOURCE
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

enum { DT_I32 = 3, DT_I64 = 4, DT_F16 = 5, DT_F32 = 6, DT_F64 = 7, DT_BF16 = 15 };
enum { OP_SUM = 0, OP_AVG = 1, OP_MIN = 3, OP_MAX = 4, OP_PREMUL_SUM = 8 };

#define ORC_OK 0
#define ORC_EINVAL 1

/* ---- 16-bit float helpers (bit-level, no compiler extensions) ---- */

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet (same rule torch's c10::BFloat16 uses) */
static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t bias = 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)((u + bias) >> 16);
}

static float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 (after rounding check below) or inf */
  if (a < 0x33000000u) return (uint16_t)sign;              /* < 2^-25 rounds to zero */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift, half;
  if (e < -14) {
    shift = (uint32_t)(13 + (-14 - e)); /* subnormal result */
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ffu);
  uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry may roll into exponent / inf: correct */
  return (uint16_t)(sign | q);
}

/* ---- element ops: core/cputhread.cc:125-148 ----
 * add = a + b; min = std::min(a,b) = (b < a) ? b : a; max = std::max(a,b) =
 * (a < b) ? b : a, with a the running destination and b the next source. */

#define DEF_FOLD(NAME, T, ADD)                                                        \
  static void NAME(T* dst, const T* src, size_t n, int op) {                           \
    size_t i;                                                                          \
    if (op == OP_SUM) {                                                                \
      for (i = 0; i < n; ++i) dst[i] = ADD(dst[i], src[i]);                            \
    } else if (op == OP_MIN) {                                                         \
      for (i = 0; i < n; ++i) dst[i] = (src[i] < dst[i]) ? src[i] : dst[i];            \
    } else {                                                                           \
      for (i = 0; i < n; ++i) dst[i] = (dst[i] < src[i]) ? src[i] : dst[i];            \
    }                                                                                  \
  }

#define FADD(a, b) ((a) + (b))
/* two's-complement wrap without signed-overflow UB */
#define I32ADD(a, b) ((int32_t)((uint32_t)(a) + (uint32_t)(b)))
#define I64ADD(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))

DEF_FOLD(fold_f32, float, FADD)
DEF_FOLD(fold_f64, double, FADD)
DEF_FOLD(fold_i32, int32_t, I32ADD)
DEF_FOLD(fold_i64, int64_t, I64ADD)

static size_t item_size(int dtype) {
  switch (dtype) {
  case DT_I32:
  case DT_F32:
    return 4;
  case DT_I64:
  case DT_F64:
    return 8;
  case DT_F16:
  case DT_BF16:
    return 2;
  default:
    return 0;
  }
}

size_t orc_item_size(int dtype) {
  return item_size(dtype);
}

/*
 * One rank's local multi-source reduction.
 *
 * Follows WorkReduceScatterCpu::reduceAdd (core/cputhread.cc:3571-3587): the
 * first source is memcpy'd into dst, every later one is folded element by
 * element with CpuReductions::reduce (:125-148).  The order of sources is the
 * reference's ipcRanks order (core/group.cc:567-570): first, first+1, ...,
 * nsrc-1, 0, ..., first-1 (core/cputhread.cc:3680-3686).
 *
 * op:
 *   SUM, MIN, MAX   as above.
 *   AVG             SUM, then every element times `scale` (the caller passes
 *                   1.0f/size), a separate rounding: core/processgroup.cc:1364-1366
 *                   (output.mul_(1.0f/size)).  Floating dtypes only.
 *   PREMUL_SUM      every source times `scale` first (its own rounding), then
 *                   SUM: core/processgroup.cc:1340-1344 (input * premulValue).
 *                   Floating dtypes only.
 *
 * 16-bit floats have no CPU path in the reference (core/cputhread.cc:99-107
 * aborts).  The rule used here is the one the build is specified to: convert
 * each source to fp32, fold in fp32 in the same order, round to nearest even
 * once at the end.  PREMUL rounds the product to the 16-bit type first (what
 * a 16-bit torch `input * f` produces); AVG rounds the sum, then rounds the
 * scaled value again (what `output.mul_` on a 16-bit tensor produces).
 * MIN/MAX compare the fp32 images and keep the winning operand's bits.
 */
int orc_reduce(const void* const* srcs, int nsrc, int first, void* dst, size_t numel, int dtype, int op,
    float scale) {
  size_t isz = item_size(dtype);
  if (!isz || nsrc < 1 || first < 0 || first >= nsrc) return ORC_EINVAL;
  if (op != OP_SUM && op != OP_AVG && op != OP_MIN && op != OP_MAX && op != OP_PREMUL_SUM) return ORC_EINVAL;
  int is_float = dtype == DT_F32 || dtype == DT_F64 || dtype == DT_F16 || dtype == DT_BF16;
  if ((op == OP_AVG || op == OP_PREMUL_SUM) && !is_float) return ORC_EINVAL;
  int fold_op = (op == OP_MIN || op == OP_MAX) ? op : OP_SUM;
  size_t i;
  int j;

  if (dtype == DT_BF16 || dtype == DT_F16) {
    float (*up)(uint16_t) = dtype == DT_BF16 ? bf16_to_f32 : f16_to_f32;
    uint16_t (*down)(float) = dtype == DT_BF16 ? f32_to_bf16 : f32_to_f16;
    uint16_t* out = (uint16_t*)dst;
    for (i = 0; i < numel; ++i) {
      const uint16_t* s0 = (const uint16_t*)srcs[first];
      uint16_t win = s0[i];
      float acc = up(s0[i]);
      if (op == OP_PREMUL_SUM) acc = up(down(acc * scale));
      for (j = 1; j < nsrc; ++j) {
        const uint16_t* s = (const uint16_t*)srcs[(first + j) % nsrc];
        float v = up(s[i]);
        if (op == OP_PREMUL_SUM) v = up(down(v * scale));
        if (fold_op == OP_SUM) {
          acc = acc + v;
        } else if (fold_op == OP_MIN) {
          if (v < acc) {
            acc = v;
            win = s[i];
          }
        } else {
          if (acc < v) {
            acc = v;
            win = s[i];
          }
        }
      }
      if (fold_op != OP_SUM) {
        out[i] = win;
      } else if (op == OP_AVG) {
        out[i] = down(up(down(acc)) * scale);
      } else {
        out[i] = down(acc);
      }
    }
    return ORC_OK;
  }

  /* 32/64-bit types: literal restatement, pass by pass. */
  void* tmp = NULL;
  if (op == OP_PREMUL_SUM) {
    tmp = malloc(numel * isz + 1);
    if (!tmp) return ORC_EINVAL;
  }
  for (j = 0; j < nsrc; ++j) {
    const void* s = srcs[(first + j) % nsrc];
    if (op == OP_PREMUL_SUM) {
      if (dtype == DT_F32) {
        for (i = 0; i < numel; ++i) ((float*)tmp)[i] = ((const float*)s)[i] * scale;
      } else {
        for (i = 0; i < numel; ++i) ((double*)tmp)[i] = ((const double*)s)[i] * (double)scale;
      }
      s = tmp;
    }
    if (j == 0) {
      memmove(dst, s, numel * isz);
    } else if (dtype == DT_F32) {
      fold_f32((float*)dst, (const float*)s, numel, fold_op);
    } else if (dtype == DT_F64) {
      fold_f64((double*)dst, (const double*)s, numel, fold_op);
    } else if (dtype == DT_I32) {
      fold_i32((int32_t*)dst, (const int32_t*)s, numel, fold_op);
    } else {
      fold_i64((int64_t*)dst, (const int64_t*)s, numel, fold_op);
    }
  }
  free(tmp);
  if (op == OP_AVG) {
    if (dtype == DT_F32) {
      for (i = 0; i < numel; ++i) ((float*)dst)[i] = ((float*)dst)[i] * scale;
    } else {
      for (i = 0; i < numel; ++i) ((double*)dst)[i] = ((double*)dst)[i] * (double)scale;
    }
  }
  return ORC_OK;
}

/*
 * All-gather chunk assembly, with the 2-D form the reference's copy-engine
 * path uses.
 *
 * Contiguous form (rows = 1, dst_shard_stride = pitch): WorkAllGatherCpu::step,
 * core/cputhread.cc:3446-3453 -- out[pitch*i .. +bytes] = in_i for every rank.
 * 2-D form: Copy2d / cuMemcpy2DAsync, core/processgroup.cc:806-820 -- `rows`
 * rows of `width` bytes, source row pitch `src_pitch`, destination row pitch
 * `dst_pitch`; shard s starts at dst + s*dst_shard_stride.
 */
int orc_gather(const void* const* srcs, int nsrc, void* dst, size_t width, size_t rows, size_t src_pitch,
    size_t dst_pitch, size_t dst_shard_stride) {
  if (nsrc < 0) return ORC_EINVAL;
  for (int s = 0; s < nsrc; ++s) {
    const char* in = (const char*)srcs[s];
    char* out = (char*)dst + (size_t)s * dst_shard_stride;
    for (size_t r = 0; r < rows; ++r) memmove(out + r * dst_pitch, in + r * src_pitch, width);
  }
  return ORC_OK;
}

/*
 * N-d box copy between two strided layouts (strides in elements).
 *
 * This is what a compile_op Copy means (core/cputhread.h:306-310: an
 * {offset, shape} box inside a tensor <-> a contiguous staging tensor) and,
 * with both sides strided, the fused form of Copy + Read + Copy
 * (core/cputhread.cc:5628-5672 moves the bytes of each Read unchanged).
 * The caller folds the box offset into the base pointers.
 */
int orc_copy_box(const void* src, void* dst, int ndim, const int64_t* shape, const int64_t* src_strides,
    const int64_t* dst_strides, int itemsize) {
  if (ndim < 0 || ndim > 16 || itemsize <= 0) return ORC_EINVAL;
  int64_t idx[16] = {0};
  int64_t total = 1;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] < 0) return ORC_EINVAL;
    total *= shape[d];
  }
  for (int64_t n = 0; n < total; ++n) {
    int64_t so = 0, doff = 0;
    for (int d = 0; d < ndim; ++d) {
      so += idx[d] * src_strides[d];
      doff += idx[d] * dst_strides[d];
    }
    memcpy((char*)dst + doff * itemsize, (const char*)src + so * itemsize, (size_t)itemsize);
    for (int d = ndim - 1; d >= 0; --d) {
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
    }
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------------
 * CPU baseline harness: the reference's CPU reduce-scatter as `nthreads`
 * rank-threads would run it on one host (one service thread per rank process,
 * core/cputhread.cc:6415-6433).  Each rank-thread r produces output chunk r:
 * memcpy of its own chunk, then for every peer in ipcRanks order a copy of the
 * peer's chunk into a temporary buffer (stand-in for process_vm_readv,
 * core/cputhread.cc:3589-3603) followed by the scalar fold loop (:3581-3585).
 *
 * inputs[p] is rank p's full input of nranks*numel elements; outputs[r] gets
 * numel elements.  Ranks 0..nthreads-1 run concurrently and stay alive, with their
 * temporaries, over all `reps` repetitions (a barrier starts each one).  Returns the
 * median over the repetitions of the wall seconds of the slowest thread (<0 on error).
 * ---------------------------------------------------------------------- */

typedef struct {
  const void* const* inputs;
  void* output;
  void* tmp;
  int rank, nranks, dtype, op, reps;
  size_t numel;
  pthread_barrier_t* bar;
  double* seconds; /* one per repetition */
} rank_job;

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* One rank's service thread: it lives for all repetitions, as the reference's does for the life
 * of the process (core/cputhread.cc:6415-6433), and keeps its temporary. */
static void* rank_thread(void* p) {
  rank_job* j = (rank_job*)p;
  size_t isz = item_size(j->dtype);
  size_t bytes = j->numel * isz;
  for (int rep = 0; rep < j->reps; ++rep) {
    pthread_barrier_wait(j->bar);
    double t0 = now_s();
    memcpy(j->output, (const char*)j->inputs[j->rank] + bytes * (size_t)j->rank, bytes);
    for (int k = 1; k < j->nranks; ++k) {
      int peer = (j->rank + k) % j->nranks;
      memcpy(j->tmp, (const char*)j->inputs[peer] + bytes * (size_t)j->rank, bytes);
      if (j->dtype == DT_F32) {
        fold_f32((float*)j->output, (const float*)j->tmp, j->numel, j->op);
      } else if (j->dtype == DT_F64) {
        fold_f64((double*)j->output, (const double*)j->tmp, j->numel, j->op);
      } else if (j->dtype == DT_I32) {
        fold_i32((int32_t*)j->output, (const int32_t*)j->tmp, j->numel, j->op);
      } else {
        fold_i64((int64_t*)j->output, (const int64_t*)j->tmp, j->numel, j->op);
      }
    }
    j->seconds[rep] = now_s() - t0;
  }
  return NULL;
}

static int cmp_double(const void* a, const void* b) {
  double x = *(const double*)a, y = *(const double*)b;
  return (x > y) - (x < y);
}

/* Returns the median over `reps` repetitions of the time of the slowest rank-thread; *best_out
 * (may be NULL) receives the fastest repetition. */
double orc_cpu_reduce_scatter_ranks(const void* const* inputs, void* const* outputs, int nranks, int nthreads,
    size_t numel, int dtype, int op, int reps, double* best_out) {
  size_t isz = item_size(dtype);
  if (!(dtype == DT_F32 || dtype == DT_F64 || dtype == DT_I32 || dtype == DT_I64)) return -1.0;
  if (op != OP_SUM && op != OP_MIN && op != OP_MAX) return -1.0;
  if (nthreads < 1 || nthreads > nranks || nthreads > 256 || reps < 1 || reps > 4096) return -1.0;
  pthread_t th[256];
  rank_job jobs[256];
  pthread_barrier_t bar;
  double* times = (double*)calloc((size_t)nthreads * (size_t)reps, sizeof(double));
  if (!times) return -1.0;
  for (int t = 0; t < nthreads; ++t) {
    jobs[t].tmp = malloc(numel * isz + 1);
    if (!jobs[t].tmp) return -1.0;
    /* the reference keeps its temporary across calls: take the page faults before the clock starts */
    memset(jobs[t].tmp, 0, numel * isz + 1);
  }
  pthread_barrier_init(&bar, NULL, (unsigned)nthreads);
  for (int t = 0; t < nthreads; ++t) {
    jobs[t].inputs = inputs;
    jobs[t].output = outputs[t];
    jobs[t].rank = t;
    jobs[t].nranks = nranks;
    jobs[t].dtype = dtype;
    jobs[t].op = op;
    jobs[t].reps = reps;
    jobs[t].numel = numel;
    jobs[t].bar = &bar;
    jobs[t].seconds = times + (size_t)t * (size_t)reps;
    pthread_create(&th[t], NULL, rank_thread, &jobs[t]);
  }
  for (int t = 0; t < nthreads; ++t) {
    pthread_join(th[t], NULL);
  }
  pthread_barrier_destroy(&bar);
  /* per repetition: the slowest thread */
  for (int rep = 0; rep < reps; ++rep) {
    double worst = 0.0;
    for (int t = 0; t < nthreads; ++t) {
      double s = times[(size_t)t * (size_t)reps + (size_t)rep];
      if (s > worst) worst = s;
    }
    times[rep] = worst; /* row 0 is overwritten only after its own entry was read */
  }
  qsort(times, (size_t)reps, sizeof(double), cmp_double);
  double median = times[reps / 2];
  if (best_out) *best_out = times[0];
  for (int t = 0; t < nthreads; ++t) free(jobs[t].tmp);
  free(times);
  return median;
}

/* Exposed so the tests can pin the 16-bit conversions against torch's. */
uint16_t orc_f32_to_bf16(float f) {
  return f32_to_bf16(f);
}
float orc_bf16_to_f32(uint16_t h) {
  return bf16_to_f32(h);
}
uint16_t orc_f32_to_f16(float f) {
  return f32_to_f16(f);
}
float orc_f16_to_f32(uint16_t h) {
  return f16_to_f32(h);
}
