/*
 * fx_oracle.c -- CPU restatement of FlagCX's reduce / slice / alltoallv
 * arithmetic.  TEST INFRASTRUCTURE ONLY: this file is the checker the GPU
 * path is compared against (tests, the smoke check, and the CPU-baseline leg
 * of the benchmark).  Nothing in the shipped library links, loads or calls it.
 *
 * Every function cites the reference source it restates (paths relative to
 * the FlagCX tree).  The reference's own headers on this path pull in an
 * un-vendored third-party header (nlohmann/json.hpp, empty submodule), so the
 * reference templates are not compiled here; the restatement is pinned by the
 * reference's known-answer tests and by independent IEEE-754 / integer
 * implementations instead.
 *
 * Pinning status per function:
 *   oracle_reduce2 sum/min/max on fp32/int32 .. reference KATs
 *       (test/unittest/service/test_reduction_ops.cpp:11-75) + numpy float32 /
 *       int32 arithmetic (independent correctly-rounded implementation).
 *   the other host types (int8, uint8, uint32, int64, uint64, fp64) ....
 *       numpy arithmetic of the same width (wrapping integers, IEEE double),
 *       extreme values and ties included.
 *   oracle_reduce_copy order ................... brute force over parenthesis-
 *       ations on non-associative tuples + numpy left fold.
 *   bf16 / fp16 widening and rounding ......... exhaustive tables against
 *       numpy float16 and a second, arithmetic (non bit-trick) rounding; fp64
 *       accumulation within 1 ulp.
 *   prod (all dtypes) ......................... PARITY UNPINNED by the
 *       reference (it rejects prod, service/bootstrap.cc:872-874); defined as
 *       acc*=x left to right and checked against numpy only.
 *   avg (all dtypes) .......................... PARITY UNPINNED by the
 *       reference (it only forwards avg to vendor libraries and rejects it on
 *       its own host path, service/bootstrap.cc:872-874); defined as the sum
 *       divided once by k (IEEE division before the final rounding; C division
 *       of the wrapped sum for integers) and checked against numpy only.
 *   oracle_reduce_copy_elem (16-bit types folded in the element type, the
 *       reference device kernel's own arithmetic) .. hand-derived cases where
 *       rounding after every addition and rounding once differ (bf16 256+1+1,
 *       fp16 2048+1+1), the order of its steps on a non-associative triple, its
 *       a > b ? a : b rule on +0 / -0 and on NaN in every position of a triple
 *       (worked out from custom_allreduce.cu:326-334 by hand); k = 2 sums equal
 *       the pinned oracle_reduce_copy (one rounding either way); every step is
 *       numpy's float16 addition for fp16.  The NaN PAYLOAD a sum produces is
 *       unpinned (the reference's comes from the GPU's converter).
 *   oracle_split / plans ...................... tiling invariants + closed
 *       forms of the reference's divisible cases.
 *   oracle_tree_reduce ........................ hand-derived associations for
 *       n = 3, 5, 6, 8 on non-associative values + the reference's closed forms.
 *   oracle_bootstrap_* (the host ring) ........ chunk table against the quoted
 *       formula's literal cases; association and operand order derived by hand
 *       from the reference loop for n = 3 and 4 on values where every other
 *       association / tie rule gives a different answer, and on NaN operands,
 *       which show which argument of each step is the local one; closed forms.
 *   oracle_pack / oracle_unpack ............... round-trip identity and the
 *       displacement arithmetic of service/bootstrap.cc:1253-1258.
 *   trigger encode/decode ..................... bit constants of
 *       include/flagcx_kernel_core.h:146-162.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* FlagCX enum values (include/flagcx.h:36-66). */
enum {
  DT_INT8 = 0, DT_UINT8 = 1, DT_INT32 = 2, DT_UINT32 = 3, DT_INT64 = 4, DT_UINT64 = 5,
  DT_FP16 = 6, DT_FP32 = 7, DT_FP64 = 8, DT_BF16 = 9
};
enum { OP_SUM = 0, OP_PROD = 1, OP_MAX = 2, OP_MIN = 3, OP_AVG = 4 };
enum { RC_OK = 0, RC_INVALID = 4, RC_UNSUPPORTED = 9 };

static int g_threads = 1;

/* Number of host threads the element loops are split over (1 = the
 * reference's single scalar loop per rank process). */
void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int oracle_get_threads(void) { return g_threads; }

/* flagcx.cc:35-66 (getFlagcxDataTypeSize). */
size_t oracle_dtype_size(int dtype) {
  switch (dtype) {
    case DT_INT8: case DT_UINT8: return 1;
    case DT_FP16: case DT_BF16: return 2;
    case DT_INT32: case DT_UINT32: case DT_FP32: return 4;
    case DT_INT64: case DT_UINT64: case DT_FP64: return 8;
    default: return 0;
  }
}

/* ---------------------------------------------------------------- 16-bit */

static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* bf16 is the top half of an fp32: widening is exact. */
float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet bit forced). */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* IEEE binary16 -> fp32, exact (subnormals normalised). */
float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1fu) return bits_f32(sign | 0x7f800000u | (man << 13));
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    int e = -1;
    do {
      man <<= 1;
      e++;
    } while (!(man & 0x400u));
    return bits_f32(sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3ffu) << 13));
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> IEEE binary16, round to nearest even, gradual underflow, overflow
 * to infinity; NaN keeps its top payload bits with the quiet bit forced. */
uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 or inf */
  if (a >= 0x38800000u) {                                  /* normal half */
    uint32_t r = a - 0x38000000u; /* rebias 127 -> 15 */
    r += 0xfffu + ((r >> 13) & 1u);
    return (uint16_t)(sign | (r >> 13)); /* carry may reach inf: correct */
  }
  if (a < 0x33000000u) return sign; /* below half of the least subnormal */
  /* subnormal half: value = m * 2^-24 with m in [0,1024] */
  uint32_t e = a >> 23;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift = 126u - e; /* 14..24 for this range */
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | q);
}

/* ------------------------------------------------------------ element ops */
/*
 * sum  : c = a + b               service/include/utils.h:697-705
 * max  : std::max(a,b) = (a<b)?b:a   utils.h:718-725 (ties and NaN keep a)
 * min  : std::min(a,b) = (b<a)?b:a   utils.h:707-715
 * prod : c = a * b               not in the reference (parity unpinned)
 * int32 sum/prod wrap modulo 2^32 (done in uint32_t; the reference's signed
 * overflow would be undefined behaviour).
 */
static inline float op_f32(float a, float b, int op) {
  switch (op) {
    case OP_AVG: /* accumulates like sum; the caller divides at the end */
    case OP_SUM: return a + b;
    case OP_PROD: return a * b;
    case OP_MAX: return (a < b) ? b : a;
    default: return (b < a) ? b : a;
  }
}
static inline int32_t op_i32(int32_t a, int32_t b, int op) {
  switch (op) {
    case OP_AVG:
    case OP_SUM: return (int32_t)((uint32_t)a + (uint32_t)b);
    case OP_PROD: return (int32_t)((uint32_t)a * (uint32_t)b);
    case OP_MAX: return (a < b) ? b : a;
    default: return (b < a) ? b : a;
  }
}

/*
 * The remaining element types of the host dispatch (utils.h:664-695): char
 * (signed on x86-64), unsigned char, uint32_t, int64_t, uint64_t, double.
 * T is the element type, W the unsigned type of the same width in which sum
 * and prod are computed so that they wrap instead of overflowing; for char the
 * reference's int promotion followed by the narrowing store gives the same
 * modulo-256 value.  max/min compare as T.
 */
#define ORACLE_INT_LOOP(T, W)                                                  \
  do {                                                                         \
    T *o = (T *)out;                                                           \
    _Pragma("omp parallel for num_threads(nt) schedule(static) if (nt > 1)")   \
    for (long long i = 0; i < n; i++) {                                        \
      T acc = ((const T *)in[first])[i];                                       \
      for (int j = 1; j < k; j++) {                                            \
        T x = ((const T *)in[(first + j) % k])[i];                             \
        switch (op) {                                                          \
          case OP_AVG:                                                         \
          case OP_SUM: acc = (T)(W)((W)acc + (W)x); break;                     \
          case OP_PROD: acc = (T)(W)((W)acc * (W)x); break;                    \
          case OP_MAX: acc = (acc < x) ? x : acc; break;                       \
          default: acc = (x < acc) ? x : acc; break;                           \
        }                                                                      \
      }                                                                        \
      o[i] = (op == OP_AVG) ? (T)(acc / (T)k) : acc;                           \
    }                                                                          \
  } while (0)

static inline double op_f64(double a, double b, int op) {
  switch (op) {
    case OP_AVG:
    case OP_SUM: return a + b;
    case OP_PROD: return a * b;
    case OP_MAX: return (a < b) ? b : a;
    default: return (b < a) ? b : a;
  }
}

static int check_args(int dtype, int op) {
  if (oracle_dtype_size(dtype) == 0) return RC_INVALID; /* utils.h:690-694 */
  if (op < OP_SUM || op > OP_AVG) return RC_INVALID;    /* bootstrap.cc:872-874 rejects prod and avg; both are this path's own */
  return RC_OK;
}

/*
 * k-way reduce-copy: acc = in[first]; then fold in[(first+j)%k], j=1..k-1,
 * left to right (adaptor/kernel/nvidia/custom_allreduce.cu:345-359).  For the
 * 16-bit types every input is widened to fp32, accumulated in fp32 and rounded
 * to the output type once; max/min return the selected input's own bits.
 * out may alias any input (each element is read from all inputs before it is
 * written).
 */
int oracle_reduce_copy(void *out, const void *const *in, int k, size_t count,
                       int dtype, int op, int first) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  if (k < 1 || first < 0 || first >= k) return RC_INVALID;
  const int nt = g_threads;
  long long n = (long long)count;
  if (dtype == DT_FP32) {
    float *o = (float *)out;
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (long long i = 0; i < n; i++) {
      float acc = ((const float *)in[first])[i];
      for (int j = 1; j < k; j++)
        acc = op_f32(acc, ((const float *)in[(first + j) % k])[i], op);
      o[i] = (op == OP_AVG) ? acc / (float)k : acc;
    }
  } else if (dtype == DT_INT32) {
    int32_t *o = (int32_t *)out;
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (long long i = 0; i < n; i++) {
      int32_t acc = ((const int32_t *)in[first])[i];
      for (int j = 1; j < k; j++)
        acc = op_i32(acc, ((const int32_t *)in[(first + j) % k])[i], op);
      o[i] = (op == OP_AVG) ? acc / k : acc;
    }
  } else if (dtype == DT_INT8) {
    ORACLE_INT_LOOP(int8_t, uint8_t);
  } else if (dtype == DT_UINT8) {
    ORACLE_INT_LOOP(uint8_t, uint8_t);
  } else if (dtype == DT_UINT32) {
    ORACLE_INT_LOOP(uint32_t, uint32_t);
  } else if (dtype == DT_INT64) {
    ORACLE_INT_LOOP(int64_t, uint64_t);
  } else if (dtype == DT_UINT64) {
    ORACLE_INT_LOOP(uint64_t, uint64_t);
  } else if (dtype == DT_FP64) {
    double *o = (double *)out;
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (long long i = 0; i < n; i++) {
      double acc = ((const double *)in[first])[i];
      for (int j = 1; j < k; j++)
        acc = op_f64(acc, ((const double *)in[(first + j) % k])[i], op);
      o[i] = (op == OP_AVG) ? acc / (double)k : acc;
    }
  } else {
    uint16_t *o = (uint16_t *)out;
    const int bf = (dtype == DT_BF16);
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (long long i = 0; i < n; i++) {
      uint16_t hb = ((const uint16_t *)in[first])[i];
      float acc = bf ? oracle_bf16_to_f32(hb) : oracle_f16_to_f32(hb);
      if (op == OP_SUM || op == OP_PROD || op == OP_AVG) {
        for (int j = 1; j < k; j++) {
          uint16_t xb = ((const uint16_t *)in[(first + j) % k])[i];
          float x = bf ? oracle_bf16_to_f32(xb) : oracle_f16_to_f32(xb);
          acc = op_f32(acc, x, op);
        }
        if (op == OP_AVG) acc = acc / (float)k;
        o[i] = bf ? oracle_f32_to_bf16(acc) : oracle_f32_to_f16(acc);
      } else {
        for (int j = 1; j < k; j++) {
          uint16_t xb = ((const uint16_t *)in[(first + j) % k])[i];
          float x = bf ? oracle_bf16_to_f32(xb) : oracle_f16_to_f32(xb);
          int take = (op == OP_MAX) ? (acc < x) : (x < acc);
          if (take) {
            acc = x;
            hb = xb;
          }
        }
        o[i] = hb;
      }
    }
  }
  return RC_OK;
}

/*
 * The reference device kernel's own arithmetic for the 16-bit types
 * (adaptor/kernel/nvidia/custom_allreduce.cu:326-361): lsa_reduce keeps the
 * accumulator in the element type, acc = reduceOp(acc, x), with
 *   sum: a + b on half / nv_bfloat16 -- the exact sum rounded to 16 bits, at
 *        every step;
 *   max: a > b ? a : b,  min: a < b ? a : b  -- on a tie or an unordered pair
 *        the later operand b is handed on.
 * Peers are folded 0, 1, .., k-1 (rotated by `first` like oracle_reduce_copy).
 * Only what that kernel's dispatch accepts (:498-518): fp16 / bf16 with sum,
 * max, min.
 */
int oracle_reduce_copy_elem(void *out, const void *const *in, int k, size_t count, int dtype, int op, int first) {
  if (dtype != DT_FP16 && dtype != DT_BF16) return RC_UNSUPPORTED;
  if (op != OP_SUM && op != OP_MAX && op != OP_MIN) return RC_UNSUPPORTED;
  if (k < 1 || first < 0 || first >= k) return RC_INVALID;
  const int bf = (dtype == DT_BF16);
  uint16_t *o = (uint16_t *)out;
  for (size_t i = 0; i < count; i++) {
    uint16_t a = ((const uint16_t *)in[first])[i];
    for (int j = 1; j < k; j++) {
      const uint16_t b = ((const uint16_t *)in[(first + j) % k])[i];
      const float x = bf ? oracle_bf16_to_f32(a) : oracle_f16_to_f32(a);
      const float y = bf ? oracle_bf16_to_f32(b) : oracle_f16_to_f32(b);
      if (op == OP_SUM) {
        /* both operands have at most 11 significant bits, so the float sum is the exact sum (or differs from it
         * far below half a 16-bit ulp) and one rounding of it is the native 16-bit addition */
        const float s = x + y;
        a = bf ? oracle_f32_to_bf16(s) : oracle_f32_to_f16(s);
      } else if (op == OP_MAX) {
        a = (x > y) ? a : b;
      } else {
        a = (x < y) ? a : b;
      }
    }
    o[i] = a;
  }
  return RC_OK;
}

/*
 * Two-input host reduce, res = a (op) b  (utils.h:697-725).  The ring callers
 * pass a = local data, b = res = received partial (bootstrap.cc:853-871); the
 * device reduce passes a = partial, b = local
 * (adaptor/kernel/nvidia/flagcx_reduce_kernel_device.cu:75-86).
 */
int oracle_reduce2(void *res, const void *a, const void *b, size_t n, int dtype,
                   int op) {
  const void *in[2] = {a, b};
  return oracle_reduce_copy(res, in, 2, n, dtype, op, 0);
}

/*
 * The reference's host path for k inputs: k-1 successive two-input passes over
 * a running partial, each reading two arrays and writing one
 * (bootstrap.cc:853-871).  acc must hold `count` elements; it ends up equal to
 * oracle_reduce_copy's output for fp32/int32 (same order, same arithmetic).
 * Used as the CPU baseline's timed loop.
 */
int oracle_host_ring_passes(void *acc, const void *const *in, int k,
                            size_t count, int dtype, int op) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  if (op == OP_AVG) return RC_INVALID; /* a mean is not a chain of two-input means */
  if (k < 1) return RC_INVALID;
  size_t bytes = count * oracle_dtype_size(dtype);
  if (k == 1) {
    memcpy(acc, in[0], bytes);
    return RC_OK;
  }
  rc = oracle_reduce2(acc, in[0], in[1], count, dtype, op);
  for (int p = 2; p < k && !rc; p++)
    rc = oracle_reduce2(acc, acc, in[p], count, dtype, op);
  return rc;
}

/* ---------------------------------------------------------- partitioning */
/*
 * Remainder-balanced split used three times, nested (rank chunk, slice,
 * red-slice): runner/uni_runner_impl.cc:100-131, 433-457, 854-866.  Offsets
 * are in elements.
 */
void oracle_split(size_t total, size_t parts, size_t idx, size_t *cnt,
                  size_t *off) {
  size_t base = total / parts, rem = total % parts;
  *cnt = base + (idx < rem ? 1 : 0);
  *off = idx * base + (idx < rem ? idx : rem);
}

/*
 * Automatic red-slice count, evaluated in single precision exactly as the
 * reference does (uni_runner_impl.cc:694-701): ceil of the chained float
 * divisions.  nredslices != 0 is returned unchanged.
 */
size_t oracle_nredslices(size_t count, int nranks, size_t nslices,
                         size_t nredslices, size_t redslicesize) {
  if (nredslices != 0) return nredslices;
  if (count == 0 || redslicesize == 0) return 1;
  float v = (float)count / nranks / nslices / redslicesize;
  return (size_t)ceilf(v);
}

/* One two-input reduce node of a plan: buffer ids + element offsets. */
typedef struct {
  int32_t step, rank;           /* ring step, owning (simulated) rank      */
  int32_t in1_buf, in2_buf;     /* 0 = sendbuff, 1 = recvbuff, 2 = scratch */
  int32_t out_buf, slice;       /* slice index s                           */
  uint64_t in1_off, in2_off, out_off, count; /* elements */
} oracle_red_node;

/*
 * Reduce nodes of the sliced ring allreduce for one rank
 * (uni_runner_impl.cc:661-1007; reduce-scatter phase :744-884).  Returns the
 * number of nodes written (nslices * (nranks-1) * nred); nodes == NULL only
 * counts.  Node order: slice-major, then step, then red-slice, as the
 * reference enumerates them.
 */
size_t oracle_plan_ring_ar(size_t count, int nranks, int rank, size_t nslices,
                           size_t nred, oracle_red_node *nodes) {
  if (nranks < 2) return 0;
  size_t w = 0;
  for (size_t s = 0; s < nslices; s++)
    for (int i = 0; i < nranks - 1; i++) {
      int rx = ((rank - i - 1) % nranks + nranks) % nranks;
      size_t ccnt, coff, scnt, soff;
      oracle_split(count, (size_t)nranks, (size_t)rx, &ccnt, &coff);
      oracle_split(ccnt, nslices, s, &scnt, &soff);
      for (size_t r = 0; r < nred; r++) {
        size_t rcnt, roff;
        oracle_split(scnt, nred, r, &rcnt, &roff);
        if (nodes) {
          oracle_red_node *n = &nodes[w];
          n->step = i;
          n->rank = rank;
          n->slice = (int32_t)s;
          n->in1_buf = 1;
          n->in2_buf = 0;
          n->out_buf = 1;
          n->in1_off = n->in2_off = n->out_off = coff + soff + roff;
          n->count = rcnt;
        }
        w++;
      }
    }
  return w;
}

/*
 * Reduce nodes of the ring reduce-scatter for one rank
 * (uni_runner_impl.cc:1009-1264): chunk c holds recvcount elements at
 * c*recvcount, partials live in a scratch buffer and the last step writes to
 * recvbuff at the slice offset (:1204-1216).
 */
size_t oracle_plan_ring_rs(size_t recvcount, int nranks, int rank,
                           size_t nslices, size_t nred, oracle_red_node *nodes) {
  if (nranks < 2) return 0;
  size_t w = 0;
  for (size_t s = 0; s < nslices; s++)
    for (int i = 0; i < nranks - 1; i++) {
      int rx = ((rank - i - 2) % nranks + nranks) % nranks;
      size_t scnt, soff;
      oracle_split(recvcount, nslices, s, &scnt, &soff);
      for (size_t r = 0; r < nred; r++) {
        size_t rcnt, roff;
        oracle_split(scnt, nred, r, &rcnt, &roff);
        if (nodes) {
          oracle_red_node *n = &nodes[w];
          n->step = i;
          n->rank = rank;
          n->slice = (int32_t)s;
          n->in1_buf = 2;
          n->in2_buf = 0;
          n->in1_off = n->in2_off = (size_t)rx * recvcount + soff + roff;
          if (i == nranks - 2) {
            n->out_buf = 1;
            n->out_off = soff + roff;
          } else {
            n->out_buf = 2;
            n->out_off = n->in1_off;
          }
          n->count = rcnt;
        }
        w++;
      }
    }
  return w;
}

/*
 * Local-reduce plan (uni_runner_impl.cc:82-157): each rank reduces its own
 * chunk slice by slice, recv = recv (op) send.
 */
size_t oracle_plan_locred(size_t count, int nranks, int rank, size_t nslices,
                          oracle_red_node *nodes) {
  if (nranks < 2) return 0;
  size_t ccnt, coff;
  oracle_split(count, (size_t)nranks, (size_t)rank, &ccnt, &coff);
  for (size_t s = 0; s < nslices; s++) {
    size_t scnt, soff;
    oracle_split(ccnt, nslices, s, &scnt, &soff);
    if (nodes) {
      oracle_red_node *n = &nodes[s];
      n->step = 0;
      n->rank = rank;
      n->slice = (int32_t)s;
      n->in1_buf = 1;
      n->in2_buf = 0;
      n->out_buf = 1;
      n->in1_off = n->in2_off = n->out_off = coff + soff;
      n->count = scnt;
    }
  }
  return nslices;
}

/*
 * Whole ring allreduce for nranks simulated ranks, hop by hop
 * (uni_runner_impl.cc:349-659 with the transport replaced by memcpy):
 * reduce-scatter step i moves chunk (r-i)%n from rank r to rank r+1, which
 * then reduces recv = recv (op) send on it; all-gather step i moves chunk
 * (r-i+1)%n.  send[r] / recv[r] are per-rank host buffers of `count` elements.
 * Steps are executed for all ranks in lock step (snapshot of what every rank
 * transmits is taken before any rank reduces).
 */
int oracle_ring_allreduce(void *const *recv, const void *const *send,
                          int nranks, size_t count, int dtype, int op) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  if (op == OP_AVG) return RC_INVALID; /* a mean is not a chain of two-input means */
  size_t ts = oracle_dtype_size(dtype);
  if (nranks < 1) return RC_INVALID;
  if (nranks == 1) {
    if (count && recv[0] != send[0]) memmove(recv[0], send[0], count * ts);
    return RC_OK;
  }
  size_t maxchunk = count / nranks + 1;
  char *wire = (char *)malloc((size_t)nranks * maxchunk * ts);
  if (!wire) return RC_INVALID;
  for (int i = 0; i < nranks - 1; i++) {
    for (int r = 0; r < nranks; r++) { /* what rank r puts on the wire */
      int tx = ((r - i) % nranks + nranks) % nranks;
      size_t c, o;
      oracle_split(count, (size_t)nranks, (size_t)tx, &c, &o);
      const char *src = (i == 0) ? (const char *)send[r] : (const char *)recv[r];
      memcpy(wire + (size_t)r * maxchunk * ts, src + o * ts, c * ts);
    }
    for (int r = 0; r < nranks; r++) {
      int prev = (r - 1 + nranks) % nranks;
      int rx = ((r - i - 1) % nranks + nranks) % nranks;
      size_t c, o;
      oracle_split(count, (size_t)nranks, (size_t)rx, &c, &o);
      char *dst = (char *)recv[r] + o * ts;
      memcpy(dst, wire + (size_t)prev * maxchunk * ts, c * ts);
      /* device reduce node: out = in1 + in2 with in1 = recv, in2 = send */
      oracle_reduce2(dst, dst, (const char *)send[r] + o * ts, c, dtype, op);
    }
  }
  for (int i = 0; i < nranks - 1; i++) {
    for (int r = 0; r < nranks; r++) {
      int tx = ((r - i + 1) % nranks + nranks) % nranks;
      size_t c, o;
      oracle_split(count, (size_t)nranks, (size_t)tx, &c, &o);
      memcpy(wire + (size_t)r * maxchunk * ts, (const char *)recv[r] + o * ts,
             c * ts);
    }
    for (int r = 0; r < nranks; r++) {
      int prev = (r - 1 + nranks) % nranks;
      int rx = ((r - i) % nranks + nranks) % nranks;
      size_t c, o;
      oracle_split(count, (size_t)nranks, (size_t)rx, &c, &o);
      memcpy((char *)recv[r] + o * ts, wire + (size_t)prev * maxchunk * ts,
             c * ts);
    }
  }
  free(wire);
  return RC_OK;
}

/*
 * Binomial ("halving doubling") tree reduce to `root`, hop by hop
 * (runner/uni_runner_impl.cc:1266-1557).  With a = (rank - root) mod n, rank a
 * receives from a + 2^i for i = 0 .. steps(a)-1 and each time computes
 * partial = received (op) partial (the reduce node's input1 is the received
 * data, :1448-1457); steps(0) = ceil(log2 n), otherwise ctz(a) clipped so that
 * a + 2^i < n (:1316-1326).  For n = 8, root 0:
 * ((x7+x6)+(x5+x4)) + ((x3+x2)+(x1+x0)).
 */
static int tree_steps(int a, int n) {
  int total = 0;
  while ((1 << total) < n) total++; /* 8*sizeof(int) - clz(n-1) for n >= 2 */
  if (a == 0) return total;
  int st = __builtin_ctz((unsigned)a);
  if (st && n - a <= (1 << (st - 1))) {
    int rest = n - a - 1;
    st = 0;
    while (rest) {
      st++;
      rest >>= 1;
    }
  }
  return st;
}

int oracle_tree_steps(int algo_rank, int nranks) { return tree_steps(algo_rank, nranks); }

static int tree_value(void *acc, const void *const *send, int n, int root, int a, size_t count, int dtype, int op) {
  size_t bytes = count * oracle_dtype_size(dtype);
  memcpy(acc, send[(a + root) % n], bytes);
  int st = tree_steps(a, n);
  for (int i = 0; i < st; i++) {
    void *peer = malloc(bytes ? bytes : 1);
    if (!peer) return RC_INVALID;
    int rc = tree_value(peer, send, n, root, a + (1 << i), count, dtype, op);
    if (!rc) rc = oracle_reduce2(acc, peer, acc, count, dtype, op); /* received (op) own */
    free(peer);
    if (rc) return rc;
  }
  return RC_OK;
}

int oracle_tree_reduce(void *recv_root, const void *const *send, int nranks, int root, size_t count, int dtype,
                       int op) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  if (op == OP_AVG) return RC_INVALID; /* a mean is not a chain of two-input means */
  if (nranks < 1 || root < 0 || root >= nranks) return RC_INVALID;
  if (nranks == 1) {
    if (count && recv_root != send[0]) memmove(recv_root, send[0], count * oracle_dtype_size(dtype));
    return RC_OK;
  }
  return tree_value(recv_root, send, nranks, root, 0, count, dtype, op);
}

/* ------------------------------------------------ host (bootstrap) ring */
/*
 * Chunking of the reference's host collectives (service/bootstrap.cc:900-922,
 * 950-972): ChunkBytes = ceil(size / n) rounded up to a whole element; chunk i
 * starts at min(i * ChunkBytes, size); the last non-empty chunk is short and
 * the ones after it are empty.  Offsets and lengths in bytes.
 */
void oracle_bootstrap_chunks(size_t size, int nranks, size_t ts, size_t *offset,
                             size_t *length) {
  size_t chunk = (size + (size_t)nranks - 1) / (size_t)nranks;
  chunk = (chunk + ts - 1) / ts * ts;
  for (size_t i = 0; i < (size_t)nranks; i++) {
    if (chunk * i >= size) {
      offset[i] = size;
      length[i] = 0;
    } else {
      offset[i] = chunk * i;
      length[i] = (chunk * (i + 1) >= size) ? size - chunk * i : chunk;
    }
  }
}

/*
 * bootstrapRingReduceScatter (service/bootstrap.cc:787-897), every rank played
 * hop by hop.  Iteration i: rank r forwards chunk (r-i-1)%n -- its own data in
 * iteration 0, what it reduced in the previous iteration afterwards -- and
 * reduces the chunk (r-i-2)%n it receives as res = local (op) received
 * (operand order of the sum/max/min calls at :853-871).  After n-1 iterations
 * rank r holds chunk r; out[r] receives those length[r] bytes.
 */
int oracle_bootstrap_reduce_scatter(void *const *out, const void *const *send,
                                    int nranks, const size_t *offset,
                                    const size_t *length, int dtype, int op) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  if (op == OP_AVG || nranks < 2) return RC_INVALID;
  const size_t ts = oracle_dtype_size(dtype);
  size_t sub = 0;
  for (int i = 0; i < nranks; i++)
    if (length[i] > sub) sub = length[i];
  /* partial[r] = what rank r reduced last (data_for_recv); flight[r] = what it sends */
  char **partial = (char **)calloc((size_t)nranks, sizeof(char *));
  char **flight = (char **)calloc((size_t)nranks, sizeof(char *));
  if (!partial || !flight) return RC_INVALID;
  for (int r = 0; r < nranks; r++) {
    partial[r] = (char *)calloc(sub ? sub : 1, 1);
    flight[r] = (char *)calloc(sub ? sub : 1, 1);
  }
  for (int iter = 0; iter < nranks - 1 && !rc; iter++) {
    for (int r = 0; r < nranks; r++) { /* everybody prepares what it sends */
      int sc = (r + 2 * nranks - iter - 1) % nranks;
      if (!length[sc]) continue;
      if (iter == 0)
        memcpy(flight[r], (const char *)send[r] + offset[sc], length[sc]);
      else
        memcpy(flight[r], partial[r], length[sc]);
    }
    for (int r = 0; r < nranks && !rc; r++) { /* receive from the previous rank and reduce */
      int rcv = (r + 2 * nranks - iter - 2) % nranks;
      if (!length[rcv]) continue;
      int prev = (r + nranks - 1) % nranks;
      memcpy(partial[r], flight[prev], length[rcv]);
      rc = oracle_reduce2(partial[r], (const char *)send[r] + offset[rcv], partial[r], length[rcv] / ts, dtype, op);
    }
  }
  for (int r = 0; r < nranks; r++) {
    if (!rc && length[r]) memcpy(out[r], partial[r], length[r]);
    free(partial[r]);
    free(flight[r]);
  }
  free(partial);
  free(flight);
  return rc;
}

/*
 * AllReduceBootstrap (service/bootstrap.cc:993-1011, 899-942): chunks as above,
 * the ring reduce-scatter, then an all-gather that moves bytes only.  recv[r]
 * may alias send[r].
 */
int oracle_bootstrap_allreduce(void *const *recv, const void *const *send,
                               int nranks, size_t count, int dtype, int op) {
  int rc = check_args(dtype, op);
  if (rc) return rc;
  const size_t ts = oracle_dtype_size(dtype), size = count * ts;
  if (nranks < 1) return RC_INVALID;
  if (nranks == 1) {
    if (size && recv[0] != send[0]) memmove(recv[0], send[0], size);
    return RC_OK;
  }
  size_t *offset = (size_t *)calloc(2 * (size_t)nranks, sizeof(size_t)), *length = offset + nranks;
  char *full = (char *)malloc(size ? size : 1);
  void **piece = (void **)calloc((size_t)nranks, sizeof(void *));
  if (!offset || !full || !piece) return RC_INVALID;
  oracle_bootstrap_chunks(size, nranks, ts, offset, length);
  for (int r = 0; r < nranks; r++) piece[r] = full + offset[r];
  rc = oracle_bootstrap_reduce_scatter(piece, send, nranks, offset, length, dtype, op);
  for (int r = 0; r < nranks && !rc; r++)
    if (size) memcpy(recv[r], full, size);
  free(piece);
  free(full);
  free(offset);
  return rc;
}

/* ------------------------------------------------------------- alltoallv */
/*
 * pack: gather npeers segments of sendbuff (element displacements sdispls,
 * element counts counts) into contiguous slots, slot_i = sum_{j<i} counts[j].
 * The segment addressing is the reference's send side
 * (service/bootstrap.cc:1253-1258; runner/uni_runner.cc:197-210).  Zero
 * counts are skipped (adaptor/include/adaptor.h:77).
 */
void oracle_pack(void *packed, const void *sendbuff, const size_t *counts,
                 const size_t *displs, int npeers, size_t elsize) {
  size_t slot = 0;
  for (int i = 0; i < npeers; i++) {
    if (counts[i])
      memcpy((char *)packed + slot * elsize,
             (const char *)sendbuff + displs[i] * elsize, counts[i] * elsize);
    slot += counts[i];
  }
}

/* unpack: the inverse scatter, recvbuff[rdispls[i] + j] = packed[slot_i + j]. */
void oracle_unpack(void *recvbuff, const void *packed, const size_t *counts,
                   const size_t *displs, int npeers, size_t elsize) {
  size_t slot = 0;
  for (int i = 0; i < npeers; i++) {
    if (counts[i])
      memcpy((char *)recvbuff + displs[i] * elsize,
             (const char *)packed + slot * elsize, counts[i] * elsize);
    slot += counts[i];
  }
}

/*
 * alltoallv among n ranks held in one address space
 * (service/bootstrap.cc:1241-1281 with send/recv replaced by memcpy): rank r's
 * segment for peer i lands in peer i's recvbuff at rdispls[i][r].
 * counts/displs are row-major [rank][peer] tables.
 */
void oracle_alltoallv(void *const *recv, const void *const *send,
                      const size_t *sendcounts, const size_t *sdispls,
                      const size_t *rdispls, int n, size_t elsize) {
  for (int r = 0; r < n; r++)
    for (int i = 0; i < n; i++) {
      size_t c = sendcounts[r * n + i];
      if (!c) continue;
      memcpy((char *)recv[i] + rdispls[i * n + r] * elsize,
             (const char *)send[r] + sdispls[r * n + i] * elsize, c * elsize);
    }
}

/* --------------------------------------------------------- reduce trigger */
/*
 * 32-byte slice descriptor: value[0..2] = in1, in2, out; value[3] packs
 * count[31:0] nthreads[47:32] datatype[51:48] redop[55:52] state[57:56]
 * (include/flagcx_kernel_core.h:146-162; core/flagcx_reduce_kernel_host.cc:6-26).
 */
void oracle_trigger_encode(uint64_t v[4], uint64_t in1, uint64_t in2,
                           uint64_t out, uint64_t count, uint64_t nthreads,
                           int dtype, int op, int state) {
  v[0] = in1;
  v[1] = in2;
  v[2] = out;
  v[3] = (count & 0xffffffffull) | ((nthreads & 0xffffull) << 32) |
         (((uint64_t)dtype & 0xfull) << 48) | (((uint64_t)op & 0xfull) << 52) |
         (((uint64_t)state & 0x3ull) << 56);
}

void oracle_trigger_decode(const uint64_t v[4], uint64_t *count,
                           uint64_t *nthreads, int *dtype, int *op,
                           int *state) {
  *count = v[3] & 0xffffffffull;
  *nthreads = (v[3] >> 32) & 0xffffull;
  *dtype = (int)((v[3] >> 48) & 0xfull);
  *op = (int)((v[3] >> 52) & 0xfull);
  *state = (int)((v[3] >> 56) & 0x3ull);
}
