/*
 * vr_oracle.c — CPU restatement of the reference all-reduce / all-gather
 * arithmetic.  TEST INFRASTRUCTURE ONLY (see vr_oracle.h): the shipped HIP path
 * never links or calls this file.
 *
 * Two independent restatements live here on purpose:
 *   1. closed-form summation orders (vro_allreduce_*), and
 *   2. message-level emulators (vro_emulate_*) that push wires through
 *      scatter/gather sinks with the reference's own index arithmetic.
 * The test-suite requires them to agree bit for bit, which is what pins the
 * orders beyond the hand-computed known-answer vectors.
 */
#include "vr_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__x86_64__)
#include <immintrin.h>
#endif

enum { MAXR = 16 };

/* ========================================================================= */
/* binary16                                                                   */
/* ========================================================================= */

uint16_t vro_f16_add_soft(uint16_t a, uint16_t b) {
  const unsigned ea = (a >> 10) & 0x1f, eb = (b >> 10) & 0x1f;
  const unsigned ma = a & 0x3ff, mb = b & 0x3ff;
  const unsigned sa = a >> 15, sb = b >> 15;

  if (ea == 31) {
    if (ma) return (uint16_t)(a | 0x200);                 /* NaN in -> quiet NaN out  */
    if (eb == 31) {
      if (mb) return (uint16_t)(b | 0x200);
      return (sa == sb) ? a : (uint16_t)0x7e00;           /* inf - inf                */
    }
    return a;
  }
  if (eb == 31) return mb ? (uint16_t)(b | 0x200) : b;

  /* Every finite binary16 is an integer multiple of 2^-24 below 2^40. */
  int64_t va = (int64_t)(ea ? (ma | 0x400) : ma) << (ea ? ea - 1 : 0);
  int64_t vb = (int64_t)(eb ? (mb | 0x400) : mb) << (eb ? eb - 1 : 0);
  if (sa) va = -va;
  if (sb) vb = -vb;
  int64_t s = va + vb;                                     /* exact                    */

  if (s == 0) return (uint16_t)((sa & sb) << 15);          /* -0 only for (-0)+(-0)    */
  const unsigned sign = s < 0;
  uint64_t mag = (uint64_t)(sign ? -s : s);

  int p = 63 - __builtin_clzll(mag);                       /* index of leading one     */
  uint32_t bits;
  if (p <= 10) {
    bits = (uint32_t)mag;                                  /* subnormal or e==1: exact */
  } else {
    const int shift = p - 10;
    uint64_t q = mag >> shift;
    const uint64_t rem = mag & ((1ull << shift) - 1);
    const uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) ++q;       /* round to nearest even    */
    bits = (uint32_t)(((uint64_t)(shift + 1) << 10) + q - 1024);  /* carry bumps exponent */
    if (bits >= 0x7c00) bits = 0x7c00;                     /* overflow -> inf          */
  }
  return (uint16_t)(bits | (sign << 15));
}

static float f16_to_f32_soft(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff, u;
  if (e == 31) {
    u = sign | 0x7f800000u | (m << 13);
  } else if (e == 0) {
    if (m == 0) {
      u = sign;
    } else {
      int lz = __builtin_clz(m) - 21;                      /* shifts to reach bit 10   */
      m = (m << lz) & 0x3ff;
      u = sign | ((uint32_t)(113 - lz) << 23) | (m << 13);
    }
  } else {
    u = sign | ((e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_f16_soft(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000);
  const uint32_t e = (u >> 23) & 0xff;
  uint32_t m = u & 0x7fffff;
  if (e == 255) return (uint16_t)(sign | 0x7c00 | (m ? (0x200 | (m >> 13)) : 0));
  int he = (int)e - 112;                                   /* rebiased exponent        */
  if (he >= 31) return (uint16_t)(sign | 0x7c00);
  if (he <= 0) {
    if (he < -10) return sign;                             /* below half the min subnormal */
    m |= 0x800000;
    const int shift = 14 - he;                             /* 14..24                   */
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) ++q;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)he << 10) | (m >> 13);
  const uint32_t rem = m & 0x1fff;
  if (rem > 0x1000 || (rem == 0x1000 && (q & 1))) ++q;     /* carry may reach inf: correct */
  return (uint16_t)(sign | q);
}

#if defined(__x86_64__)
__attribute__((target("f16c"))) static float f16_to_f32_hw(uint16_t h) { return _cvtsh_ss(h); }
__attribute__((target("f16c"))) static uint16_t f32_to_f16_hw(float f) {
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}
static int have_f16c(void) {
  static int cached = -1;
  if (cached < 0) cached = __builtin_cpu_supports("f16c") ? 1 : 0;
  return cached;
}
#else
static int have_f16c(void) { return 0; }
static float f16_to_f32_hw(uint16_t h) { return f16_to_f32_soft(h); }
static uint16_t f32_to_f16_hw(float f) { return f32_to_f16_soft(f); }
#endif

float vro_f16_to_f32(uint16_t h) { return have_f16c() ? f16_to_f32_hw(h) : f16_to_f32_soft(h); }
uint16_t vro_f32_to_f16(float f) { return have_f16c() ? f32_to_f16_hw(f) : f32_to_f16_soft(f); }

/* Entry points that let the tests compare the two conversion routes directly. */
float vro_f16_to_f32_soft(uint16_t h) { return f16_to_f32_soft(h); }
uint16_t vro_f32_to_f16_soft(float f) { return f32_to_f16_soft(f); }

uint16_t vro_f16_add(uint16_t a, uint16_t b) {
  return vro_f32_to_f16(vro_f16_to_f32(a) + vro_f16_to_f32(b));
}

static inline int is_nan16(uint16_t h) { return (h & 0x7c00) == 0x7c00 && (h & 0x3ff); }

int vro_f16_same(uint16_t a, uint16_t b) { return a == b || (is_nan16(a) && is_nan16(b)); }

/* bfloat16: the upper half of a binary32.  Sum in binary32 (exact inputs, one
 * rounding), then round to nearest even on the 16 dropped bits; NaN stays NaN. */
uint16_t vro_bf16_add(uint16_t a, uint16_t b) {
  uint32_t ua = (uint32_t)a << 16, ub = (uint32_t)b << 16, us;
  float fa, fb, fs;
  memcpy(&fa, &ua, 4);
  memcpy(&fb, &ub, 4);
  fs = fa + fb;
  memcpy(&us, &fs, 4);
  if ((us & 0x7f800000u) == 0x7f800000u && (us & 0x007fffffu)) return (uint16_t)((us >> 16) | 0x0040);
  us += 0x7fffu + ((us >> 16) & 1u);
  return (uint16_t)(us >> 16);
}

static inline int is_nan_bf16(uint16_t h) { return (h & 0x7f80) == 0x7f80 && (h & 0x7f); }

/* Hot inner add for the order loops.  The float route when F16C exists (fast),
 * else the integer route; both give identical bits for non-NaN results. */
#if defined(__x86_64__)
__attribute__((target("f16c"))) static inline uint16_t add_hw(uint16_t a, uint16_t b) {
  return _cvtss_sh(_cvtsh_ss(a) + _cvtsh_ss(b), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}
#endif

/* Exhaustive / strided agreement check between the integer add and the float
 * add.  Returns the number of (a,b) pairs whose results differ (NaN == NaN);
 * first_bad receives a<<16|b of the first difference. */
uint64_t vro_selftest_add(uint32_t stride_a, uint32_t stride_b, uint32_t *first_bad) {
  uint64_t bad = 0;
  uint32_t first = 0xffffffffu;
  if (stride_a == 0) stride_a = 1;
  if (stride_b == 0) stride_b = 1;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : bad) reduction(min : first)
  for (uint32_t a = 0; a < 0x10000; a += stride_a) {
    for (uint32_t b = 0; b < 0x10000; b += stride_b) {
      uint16_t s = vro_f16_add_soft((uint16_t)a, (uint16_t)b);
      uint16_t f = vro_f16_add((uint16_t)a, (uint16_t)b);
      if (!vro_f16_same(s, f)) {
        ++bad;
        uint32_t key = (a << 16) | b;
        if (key < first) first = key;
      }
    }
  }
  if (first_bad) *first_bad = first;
  return bad;
}

/* ========================================================================= */
/* fixtures and generators                                                    */
/* ========================================================================= */

void vro_fill_pattern(uint16_t *buf, int rank, size_t n) {
  for (size_t i = 0; i < n; ++i) buf[i] = vro_f32_to_f16((float)((int)(i % 32) * (rank + 1)));
}

static inline uint64_t splitmix64_at(uint64_t seed, uint64_t k) {
  uint64_t z = seed + (k + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

/* double -> binary16 with a single RNE rounding: go through the integer grid. */
static uint16_t f64_to_f16(double d) {
  if (d != d) return 0x7e00;
  const uint16_t sign = signbit(d) ? 0x8000 : 0;
  double a = fabs(d);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00);
  if (a == 0.0) return sign;
  int ex;
  (void)frexp(a, &ex);                    /* a = f * 2^ex, f in [0.5,1) */
  int e = ex - 1;                         /* a in [2^e, 2^(e+1)) */
  if (e < -14) e = -14;                   /* subnormal grid */
  /* grid spacing 2^(e-10) */
  double scaled = ldexp(a, 10 - e);       /* exact; in [0, 2048) */
  double r = nearbyint(scaled);           /* default rounding mode = RNE */
  uint32_t q = (uint32_t)r;               /* 0..2048 */
  uint32_t bits = (e == -14 && q < 1024) ? q : (((uint32_t)(e + 15) << 10) + q - 1024);
  if (bits >= 0x7c00) bits = 0x7c00;
  return (uint16_t)(sign | bits);
}

uint16_t vro_f64_to_f16(double d) { return f64_to_f16(d); }

/* double -> bfloat16 with one rounding (8 significant bits, binary32's exponent range). */
uint16_t vro_f64_to_bf16(double d) {
  if (d != d) return 0x7fc0;
  const uint16_t sign = signbit(d) ? 0x8000 : 0;
  const double a = fabs(d);
  if (a == 0.0) return sign;
  if (a >= 0x1.ffp127) return (uint16_t)(sign | 0x7f80);   /* halfway to 2^128 and beyond -> inf */
  int ex;
  (void)frexp(a, &ex);
  int e = ex - 1;
  if (e < -126) e = -126;                                   /* subnormal grid */
  const uint32_t q = (uint32_t)nearbyint(ldexp(a, 7 - e)); /* 0..256 */
  uint32_t bits = (e == -126 && q < 128) ? q : (((uint32_t)(e + 127) << 7) + q - 128);
  if (bits >= 0x7f80) bits = 0x7f80;
  return (uint16_t)(sign | bits);
}

void vro_fill_pattern_dt(int dtype, uint16_t *buf, int rank, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    const double v = (double)((int)(i % 32) * (rank + 1));
    buf[i] = dtype == VRO_BF16 ? vro_f64_to_bf16(v) : f64_to_f16(v);
  }
}

static void generate_impl(int dtype, uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1);

void vro_generate(uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1) {
  generate_impl(VRO_F16, buf, n, seed, dist, p0, p1);
}
void vro_generate_dt(int dtype, uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1) {
  generate_impl(dtype, buf, n, seed, dist, p0, p1);
}

static void generate_impl(int dtype, uint16_t *buf, size_t n, uint64_t seed, int dist, double p0, double p1) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    const uint64_t z0 = splitmix64_at(seed, 2 * (uint64_t)i);
    const uint64_t z1 = splitmix64_at(seed, 2 * (uint64_t)i + 1);
    double x;
    if (dist == VRO_DIST_UNIFORM) {
      const double u = (double)(z0 >> 11) * 0x1.0p-53;
      x = p0 + (p1 - p0) * u;
    } else {
      const double u1 = (double)((z0 >> 11) + 1) * 0x1.0p-53;  /* (0,1] */
      const double u2 = (double)(z1 >> 11) * 0x1.0p-53;        /* [0,1) */
      x = p0 + p1 * (sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2));
    }
    buf[i] = dtype == VRO_BF16 ? vro_f64_to_bf16(x) : f64_to_f16(x);
  }
}

/* ========================================================================= */
/* chunking                                                                   */
/* ========================================================================= */

int vro_calc_work_size(uintptr_t input_addr, size_t bytes, int nchunks, size_t msg_bytes,
                       size_t *work_bytes) {
  if (input_addr % msg_bytes != 0) return VRO_ERR_UNALIGNED;
  const size_t msgs = (bytes + msg_bytes - 1) / msg_bytes;
  const size_t chunk = (msgs + (size_t)nchunks - 1) / (size_t)nchunks;
  if (msgs * msg_bytes != bytes || chunk * msg_bytes * (size_t)nchunks > bytes) return VRO_ERR_UNEVEN;
  if (work_bytes) *work_bytes = chunk * msg_bytes;
  return VRO_OK;
}

/* ========================================================================= */
/* closed-form summation orders                                               */
/* ========================================================================= */

int vro_set_threads(int nthreads) {
#ifdef _OPENMP
  if (nthreads > 0) omp_set_num_threads(nthreads);
  return omp_get_max_threads();
#else
  (void)nthreads;
  return 1;
#endif
}

#define ORDER_BODY(ADD)                                                             \
  do {                                                                              \
    if (mode == 0) {                                                                \
      _Pragma("omp parallel for schedule(static)") for (size_t i = 0; i < n; ++i) { \
        uint16_t s = 0; /* +0.0, as `T sum = 0.0` */                                 \
        for (int r = 0; r < nranks; ++r) s = ADD(s, in[r][i]);                      \
        out[i] = s;                                                                 \
      }                                                                             \
    } else if (mode == 1) {                                                         \
      const size_t chunk = n / (size_t)nranks;                                      \
      _Pragma("omp parallel for schedule(static)") for (size_t i = 0; i < n; ++i) { \
        const int c = (int)(i / chunk);                                             \
        uint16_t s = in[c][i];                                                      \
        for (int k = 1; k < nranks; ++k) s = ADD(in[(c + k) % nranks][i], s);       \
        out[i] = s;                                                                 \
      }                                                                             \
    } else {                                                                        \
      const size_t chunk = n / (size_t)nranks;                                      \
      const int half = nranks / 2;                                                  \
      _Pragma("omp parallel for schedule(static)") for (size_t i = 0; i < n; ++i) { \
        const int c = (int)(i / chunk);                                             \
        const int h = c / half, l = c % half;                                       \
        /* Owner rank 2l+h adds its pair's far-scatter message to its own data. */  \
        uint16_t s = ADD(in[(2 * l + h) ^ 1][i], in[2 * l + h][i]);                 \
        for (int k = 1; k < half; ++k) {                                            \
          const int j = (l + k) % half;                                             \
          /* Rank 2j+h formed this pair sum the same way before scattering it. */   \
          const uint16_t p = ADD(in[(2 * j + h) ^ 1][i], in[2 * j + h][i]);         \
          s = ADD(p, s);                                                            \
        }                                                                           \
        out[i] = s;                                                                 \
      }                                                                             \
    }                                                                               \
  } while (0)

static void order_soft(int mode, uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
  ORDER_BODY(vro_f16_add_soft);
}
#if defined(__x86_64__)
__attribute__((target("f16c"))) static void order_hw(int mode, uint16_t *out,
                                                      const uint16_t *const in[], int nranks,
                                                      size_t n) {
  ORDER_BODY(add_hw);
}
#endif

static void order_bf16(int mode, uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
  ORDER_BODY(vro_bf16_add);
}

static int order_shape_ok(int mode, int nranks, size_t n);

int vro_allreduce_order_dt(int dtype, int mode, uint16_t *out, const uint16_t *const in[], int nranks,
                           size_t n) {
  if (mode < 0 || mode > 2 || !order_shape_ok(mode, nranks, n)) return -2;
  if (n == 0) return 0;
  if (dtype == VRO_BF16) order_bf16(mode, out, in, nranks, n);
  else order_soft(mode, out, in, nranks, n);
  return 0;
}

static int order_shape_ok(int mode, int nranks, size_t n) {
  if (nranks < 1 || nranks > MAXR) return 0;
  if (mode == 0) return 1;
  if (n % (size_t)nranks) return 0;
  if (mode == 2 && (nranks < 4 || (nranks & 1))) return 0;
  return 1;
}

static int order_dispatch(int mode, uint16_t *out, const uint16_t *const in[], int nranks,
                          size_t n) {
  if (!order_shape_ok(mode, nranks, n)) return -2;
  if (n == 0) return 0;
#if defined(__x86_64__)
  if (have_f16c()) {
    order_hw(mode, out, in, nranks, n);
    return 0;
  }
#endif
  order_soft(mode, out, in, nranks, n);
  return 0;
}

int vro_allreduce_rank_order(uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
  return order_dispatch(0, out, in, nranks, n);
}
int vro_allreduce_rotated(uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
  return order_dispatch(1, out, in, nranks, n);
}
int vro_allreduce_bisect(uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
  return order_dispatch(2, out, in, nranks, n);
}

/* Same three orders through the integer-only add (slow; used to cross-check). */
int vro_allreduce_order_soft(int mode, uint16_t *out, const uint16_t *const in[], int nranks,
                             size_t n) {
  if (!order_shape_ok(mode, nranks, n)) return -2;
  if (n) order_soft(mode, out, in, nranks, n);
  return 0;
}

void vro_allgather(uint16_t *out, const uint16_t *const in[], int nranks, size_t n) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < nranks; ++r) memcpy(out + (size_t)r * n, in[r], n * sizeof(uint16_t));
}

size_t vro_count_mismatch_dt(int dtype, const uint16_t *a, const uint16_t *b, size_t n) {
  size_t bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
  for (size_t i = 0; i < n; ++i)
    bad += dtype == VRO_BF16 ? !(a[i] == b[i] || (is_nan_bf16(a[i]) && is_nan_bf16(b[i])))
                             : !vro_f16_same(a[i], b[i]);
  return bad;
}

size_t vro_count_mismatch(const uint16_t *a, const uint16_t *b, size_t n) {
  size_t bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
  for (size_t i = 0; i < n; ++i) bad += !vro_f16_same(a[i], b[i]);
  return bad;
}

/* ========================================================================= */
/* message-level emulators                                                    */
/* ========================================================================= */

enum { SG = 16, MSG_DW = 32, MSG_BYTES = 128, NSLOT_PAR = 8, MAXLAUNCH = 4096 };

typedef struct {
  int cap_dw;    /* payload dwords per wire                     */
  int wire;      /* VRO_WIRE_*                                   */
} wire_fmt;

/* Payload dwords per wire and the per-lane load shape (lanes that load x dwords each):
 * Rt64 16 x 1 (rt64.hpp:339,566-583), Rt64_128 15 x 2 (rt64_128.hpp:551,563-583),
 * Rt64_PCIE 16 x 2 (rt64.hpp:8,26-31), Rt64_128_PCIE 15 x 4 (rt64_128.hpp:14-21,33-52). */
enum { MAX_DW = 64 };
static int fmt_lanes(int wire) { return (wire == VRO_WIRE_RT64 || wire == VRO_WIRE_RT64_PCIE) ? 16 : 15; }
static int fmt_dw_per_lane(int wire) {
  switch (wire) {
    case VRO_WIRE_RT64: return 1;
    case VRO_WIRE_RT64_128: return 2;
    case VRO_WIRE_RT64_PCIE: return 2;
    default: return 4;
  }
}
static int fmt_is_pcie(int wire) { return wire == VRO_WIRE_RT64_PCIE || wire == VRO_WIRE_RT64_128_PCIE; }

static wire_fmt make_fmt(int wire) {
  wire_fmt f;
  f.wire = wire;
  f.cap_dw = fmt_lanes(wire) * fmt_dw_per_lane(wire);
  return f;
}

/* Dwords of one message: 128 bytes (Rt64, Rt64_128) or 256 bytes (the *_PCIE formats). */
static int fmt_msg_dw(int wire) { return fmt_is_pcie(wire) ? 64 : 32; }

/* Pack `cap_dw` payload dwords + flag into one message, byte for byte as the device
 * code of the reference lays it out at sub-group size 16 (lane l owns dwords
 * [l * k, l * k + k) of the message, k = dwords per lane):
 * RT64         : lane l stores {data_l, flag}: dwords 2l, 2l+1 (rt64.hpp:335-337, 566-583).
 * RT64_PCIE    : lane l stores {d_2l, d_2l+1, flag, flag}: dwords 4l .. 4l+3 (rt64.hpp:3-20,
 *                61-98: insertFlags writes the last two components of every lane).
 * RT64_128     : dwords 0..14, 16..29 payload in place, payload dword 15 parked at 30,
 *                flag at dwords 15 and 31 (rt64_128.hpp:544-553, 635-685, 724-762; the dead
 *                verifier agrees: temp[30] = temp[15]; temp[15] = flag; temp[31] = flag,
 *                allreduce.cpp:71, 131-133).
 * RT64_128_PCIE: 60 payload dwords; flag in the last component of lanes 3, 7, 11, 15 =
 *                dwords 15, 31, 47, 63; the payload dwords displaced from 15, 31, 47 are
 *                parked in lane 15's components 0, 1, 2 = dwords 60, 61, 62
 *                (rt64_128.hpp:7-13, 101-117, 194-203). */
static void pack_msg(const wire_fmt *f, uint32_t *msg, const uint32_t *payload, uint32_t flag) {
  switch (f->wire) {
    case VRO_WIRE_RT64:
      for (int l = 0; l < SG; ++l) {
        msg[2 * l] = payload[l];
        msg[2 * l + 1] = flag;
      }
      break;
    case VRO_WIRE_RT64_PCIE:
      for (int l = 0; l < SG; ++l) {
        msg[4 * l] = payload[2 * l];
        msg[4 * l + 1] = payload[2 * l + 1];
        msg[4 * l + 2] = flag;
        msg[4 * l + 3] = flag;
      }
      break;
    case VRO_WIRE_RT64_128:
      for (int k = 0; k < 30; ++k) msg[k] = payload[k];
      msg[30] = payload[15];
      msg[15] = flag;
      msg[31] = flag;
      break;
    default:
      for (int k = 0; k < 60; ++k) msg[k] = payload[k];
      msg[60] = payload[15];
      msg[61] = payload[31];
      msg[62] = payload[47];
      msg[15] = msg[31] = msg[47] = msg[63] = flag;
      break;
  }
}

/* Returns 0 and the payload when every flag position matches, else -1. */
static int unpack_msg(const wire_fmt *f, const uint32_t *msg, uint32_t *payload, uint32_t flag) {
  switch (f->wire) {
    case VRO_WIRE_RT64:
      for (int l = 0; l < SG; ++l) {
        if (msg[2 * l + 1] != flag) return -1;
        payload[l] = msg[2 * l];
      }
      break;
    case VRO_WIRE_RT64_PCIE:
      for (int l = 0; l < SG; ++l) {
        if (msg[4 * l + 2] != flag || msg[4 * l + 3] != flag) return -1;
        payload[2 * l] = msg[4 * l];
        payload[2 * l + 1] = msg[4 * l + 1];
      }
      break;
    case VRO_WIRE_RT64_128:
      if (msg[15] != flag || msg[31] != flag) return -1;
      for (int k = 0; k < 30; ++k) payload[k] = msg[k];
      payload[15] = msg[30];
      break;
    default:
      if (msg[15] != flag || msg[31] != flag || msg[47] != flag || msg[63] != flag) return -1;
      for (int k = 0; k < 60; ++k) payload[k] = msg[k];
      payload[15] = msg[60];
      payload[31] = msg[61];
      payload[47] = msg[62];
      break;
  }
  return 0;
}

int vro_wire_payload_dwords(int wire) {
  return (wire < VRO_WIRE_RT64 || wire > VRO_WIRE_RT64_128_PCIE) ? -1 : make_fmt(wire).cap_dw;
}
int vro_wire_message_dwords(int wire) {
  return (wire < VRO_WIRE_RT64 || wire > VRO_WIRE_RT64_128_PCIE) ? -1 : fmt_msg_dw(wire);
}
int vro_pack_message(int wire, uint32_t *msg, const uint32_t *payload, uint32_t flag) {
  if (wire < VRO_WIRE_RT64 || wire > VRO_WIRE_RT64_128_PCIE) return -2;
  const wire_fmt f = make_fmt(wire);
  pack_msg(&f, msg, payload, flag);
  return 0;
}
int vro_unpack_message(int wire, const uint32_t *msg, uint32_t *payload, uint32_t flag) {
  if (wire < VRO_WIRE_RT64 || wire > VRO_WIRE_RT64_128_PCIE) return -2;
  const wire_fmt f = make_fmt(wire);
  return unpack_msg(&f, msg, payload, flag);
}

/* A sink cell of the ring / sequential emulators: one packed message. */
typedef struct {
  uint32_t msg[64];
} cell;
static void cell_send(const wire_fmt *f, cell *c, const uint32_t *payload, uint32_t flag) {
  pack_msg(f, c->msg, payload, flag);
}
static int cell_recv(const wire_fmt *f, const cell *c, uint32_t *payload, uint32_t flag) {
  memset(payload, 0, sizeof(uint32_t) * MAX_DW);
  return unpack_msg(f, c->msg, payload, flag);
}

/* Predicated load of one wire: lanes whose first element index is >= n_left stay 0. */
static void load_wire(const wire_fmt *f, uint32_t *payload, const uint16_t *src, size_t n_left) {
  const int lanes = fmt_lanes(f->wire);
  const int dw_per_lane = fmt_dw_per_lane(f->wire);
  memset(payload, 0, sizeof(uint32_t) * MAX_DW);
  for (int l = 0; l < lanes; ++l) {
    const size_t off = (size_t)l * dw_per_lane * 2;       /* in halves */
    if (off < n_left) memcpy(payload + l * dw_per_lane, src + off, 4u * dw_per_lane);
  }
}

static void store_wire(const wire_fmt *f, uint16_t *dst, const uint32_t *payload, size_t n_left) {
  const int lanes = fmt_lanes(f->wire);
  const int dw_per_lane = fmt_dw_per_lane(f->wire);
  for (int l = 0; l < lanes; ++l) {
    const size_t off = (size_t)l * dw_per_lane * 2;
    if (off < n_left) memcpy(dst + off, payload + l * dw_per_lane, 4u * dw_per_lane);
  }
}

/* Element type of the emulators' adds; the *_dt entry points set it for one call.
 * (The emulators are single-threaded test helpers.) */
static int g_emul_dtype = VRO_F16;
static inline uint16_t emul_add(uint16_t a, uint16_t b) {
  return g_emul_dtype == VRO_BF16 ? vro_bf16_add(a, b) : vro_f16_add_soft(a, b);
}

/* v = m + v, element-wise in T (received message is the left operand). */
static void accum(uint32_t *v, const uint32_t *m, int ndw) {
  for (int k = 0; k < ndw; ++k) {
    const uint16_t lo = emul_add((uint16_t)(m[k] & 0xffff), (uint16_t)(v[k] & 0xffff));
    const uint16_t hi = emul_add((uint16_t)(m[k] >> 16), (uint16_t)(v[k] >> 16));
    v[k] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
}

int vro_emulate_parallel(uint16_t *const io[], int nranks, size_t n, int wire_kind, int groups,
                         int subgroups, uint32_t seq_no) {
  const int N = nranks;
  if (N < 2 || N > MAXR || n % (size_t)N || fmt_is_pcie(wire_kind)) return -2;
  const wire_fmt f = make_fmt(wire_kind);
  const size_t W = (size_t)groups * (size_t)subgroups;       /* sub-groups in the launch */
  if (W < (size_t)N || W % (size_t)N || W > MAXLAUNCH) return -3;  /* reference would spin / overrun */
  const size_t work_elems = n / (size_t)N;
  const size_t work_bytes = work_elems * 2;
  const size_t cap = (size_t)f.cap_dw * 4;
  const size_t cols = W / (size_t)N;
  const size_t loop = cols * cap;                             /* allreduce.hpp:89         */
  const size_t ring_dw = (size_t)NSLOT_PAR * MSG_DW;          /* ringSize in dwords       */

  /* One scatter and one gather buffer per rank, indexed [wire][slot][dword]. */
  const size_t buf_dw = (W + (size_t)N) * ring_dw;
  uint32_t *scat[MAXR], *gath[MAXR];
  for (int r = 0; r < N; ++r) {
    scat[r] = calloc(buf_dw, 4);
    gath[r] = calloc(buf_dw, 4);
  }
  uint32_t(*regs)[MAX_DW] = malloc(sizeof(uint32_t[MAX_DW]) * (size_t)N * (size_t)N);
  int rc = 0;

  size_t t = 0;
  for (size_t goff = 0; goff < work_bytes && rc == 0; goff += loop, ++t) {
    const uint32_t flag = seq_no + (uint32_t)(t / NSLOT_PAR);
    const size_t slot = t % NSLOT_PAR;
    for (size_t x = 0; x < cols && rc == 0; ++x) {
      const size_t wire_off = x * cap + goff;
      if (wire_off >= work_bytes) continue;                   /* workLeft <= 0           */
      const size_t off_el = wire_off / 2, left = work_elems - off_el;
      const size_t x_id = x * (size_t)N;
      uint32_t msg[32], tmp[MAX_DW];
      /* Phase A: every rank's sub-group y loads chunk y; non-owners scatter. */
      for (int r = 0; r < N; ++r)
        for (int y = 0; y < N; ++y) {
          uint32_t *v = regs[r * N + y];
          load_wire(&f, v, io[r] + (size_t)y * work_elems + off_el, left);
          if (y != r) {
            pack_msg(&f, msg, v, flag);
            memcpy(scat[y] + (x_id + (size_t)r) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
          }
        }
      /* Phase B: owner sub-group (y == r) polls peers in order r+1, r+2, ... */
      for (int r = 0; r < N && rc == 0; ++r) {
        uint32_t *v = regs[r * N + r];
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          if (unpack_msg(&f, scat[r] + (x_id + (size_t)next) * ring_dw + slot * MSG_DW, tmp, flag)) {
            rc = -1;
            break;
          }
          accum(v, tmp, f.cap_dw);
        }
        pack_msg(&f, msg, v, flag);
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          memcpy(gath[next] + (x_id + (size_t)r) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
        }
      }
      /* Phase C: non-owners poll their gather sink at [wireId = x_id + y]; all store. */
      for (int r = 0; r < N && rc == 0; ++r)
        for (int y = 0; y < N; ++y) {
          uint32_t *v = regs[r * N + y];
          if (y != r &&
              unpack_msg(&f, gath[r] + (x_id + (size_t)y) * ring_dw + slot * MSG_DW, v, flag)) {
            rc = -1;
            break;
          }
          store_wire(&f, io[r] + (size_t)y * work_elems + off_el, v, left);
        }
    }
  }
  for (int r = 0; r < N; ++r) {
    free(scat[r]);
    free(gath[r]);
  }
  free(regs);
  return rc;
}

int vro_emulate_ring(uint16_t *const io[], int nranks, size_t n, int wire_kind, int groups,
                     int subgroups, uint32_t seq_no) {
  const int N = nranks;
  if (N < 2 || N > MAXR || (N & (N - 1)) || n % (size_t)N) return -2;  /* uint32 wrap needs 2^k */
  const wire_fmt f = make_fmt(wire_kind);
  const size_t W = (size_t)groups * (size_t)subgroups;       /* parallel_sg = 1          */
  if (W == 0 || W > MAXLAUNCH) return -3;
  const size_t work_elems = n / (size_t)N, work_bytes = work_elems * 2;
  const size_t cap = (size_t)f.cap_dw * 4;
  const size_t loop = W * cap;
  enum { NSLOT = 4 };
  /* sinks: [rank][peer][slot][wire] of packed messages */
  const size_t cells = (size_t)N * NSLOT * W;
  cell *scat[MAXR], *gath[MAXR];
  for (int r = 0; r < N; ++r) {
    scat[r] = calloc(cells, sizeof(cell));
    gath[r] = calloc(cells, sizeof(cell));
  }
#define CELL(buf, peer, slot, w) ((buf) + (((size_t)(peer) * NSLOT + (slot)) * W + (w)))
  int rc = 0;
  size_t t = 0;
  for (size_t goff = 0; goff < work_bytes && rc == 0; goff += loop, ++t) {
    const uint32_t flag = seq_no + (uint32_t)(t / NSLOT);
    const size_t slot = (seq_no + t) % NSLOT;
    for (size_t w = 0; w < W && rc == 0; ++w) {
      const size_t wire_off = w * cap + goff;
      if (wire_off >= work_bytes) continue;
      const size_t off_el = wire_off / 2, left = work_elems - off_el;
      uint32_t v[MAX_DW];
      /* step 0: rank r sends chunk r to r+1 */
      for (int r = 0; r < N; ++r) {
        const int peer = r, next = (r + 1) % N;
        load_wire(&f, v, io[r] + (size_t)peer * work_elems + off_el, left);
        cell_send(&f, CELL(scat[next], peer, slot, w), v, flag);
      }
      /* steps 1..N-2: load chunk (r-i), add what (r-1) sent, forward */
      for (int i = 1; i < N - 1 && rc == 0; ++i)
        for (int r = 0; r < N; ++r) {
          const int peer = (r + N - i) % N, next = (r + 1) % N;
          cell *src = CELL(scat[r], peer, slot, w);
          uint32_t m[MAX_DW];
          if (cell_recv(&f, src, m, flag)) { rc = -1; break; }
          load_wire(&f, v, io[r] + (size_t)peer * work_elems + off_el, left);
          accum(v, m, f.cap_dw);
          memset(src, 0, sizeof *src);                        /* consumed */
          cell_send(&f, CELL(scat[next], peer, slot, w), v, flag);
        }
      /* step N-1: final add for chunk (r+1), push into the gather ring, store */
      for (int r = 0; r < N && rc == 0; ++r) {
        const int peer = (r + 1) % N, next = (r + 1) % N;
        uint32_t m[MAX_DW];
        if (cell_recv(&f, CELL(scat[r], peer, slot, w), m, flag)) { rc = -1; break; }
        load_wire(&f, v, io[r] + (size_t)peer * work_elems + off_el, left);
        accum(v, m, f.cap_dw);
        cell_send(&f, CELL(gath[next], peer, slot, w), v, flag);
        store_wire(&f, io[r] + (size_t)peer * work_elems + off_el, v, left);
      }
      /* N-2 forward+store hops, then a last store */
      for (int i = 1; i < N && rc == 0; ++i)
        for (int r = 0; r < N; ++r) {
          const int peer = (r + 1 + N - i) % N, next = (r + 1) % N;   /* p_idx = -(N-1)-i */
          uint32_t m[MAX_DW];
          if (cell_recv(&f, CELL(gath[r], peer, slot, w), m, flag)) { rc = -1; break; }
          if (i < N - 1) cell_send(&f, CELL(gath[next], peer, slot, w), m, flag);
          store_wire(&f, io[r] + (size_t)peer * work_elems + off_el, m, left);
        }
    }
  }
#undef CELL
  for (int r = 0; r < N; ++r) {
    free(scat[r]);
    free(gath[r]);
  }
  return rc;
}


/* SequentialTransmit::run (sequential_transmit.hpp:57-81, 83-207): one sub-group per
 * wire does everything its rank owes the wire.  Sinks are indexed
 * [sender's region][slot][wire] (the ringPtr typedef, l.54, indexed [tStep%nSlot][wireId]). */
int vro_emulate_sequential(uint16_t *const io[], int nranks, size_t n, int wire_kind, int groups,
                           int subgroups, uint32_t seq_no) {
  const int N = nranks;
  if (N < 2 || N > MAXR || n % (size_t)N) return -2;
  const wire_fmt f = make_fmt(wire_kind);
  const size_t W = (size_t)groups * (size_t)subgroups;       /* parallel_sg = 1          */
  if (W == 0 || W > MAXLAUNCH) return -3;
  const size_t work_elems = n / (size_t)N, work_bytes = work_elems * 2;
  const size_t cap = (size_t)f.cap_dw * 4;
  const size_t loop = W * cap;
  enum { NSLOT = 4 };
  const size_t cells = (size_t)N * NSLOT * W;
  cell *scat[MAXR], *gath[MAXR];
  for (int r = 0; r < N; ++r) {
    scat[r] = calloc(cells, sizeof(cell));
    gath[r] = calloc(cells, sizeof(cell));
  }
#define CELL(buf, region, slot, w) ((buf) + (((size_t)(region) * NSLOT + (slot)) * W + (w)))
  int rc = 0;
  size_t t = 0;
  for (size_t goff = 0; goff < work_bytes && rc == 0; goff += loop, ++t) {
    const uint32_t flag = seq_no + (uint32_t)(t / NSLOT);
    const size_t slot = t % NSLOT;
    for (size_t w = 0; w < W && rc == 0; ++w) {
      const size_t wire_off = w * cap + goff;
      if (wire_off >= work_bytes) continue;
      const size_t off_el = wire_off / 2, left = work_elems - off_el;
      /* scatter: rank r sends chunk `next` into next's sink, region r (l.96-117) */
      for (int r = 0; r < N; ++r)
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          uint32_t p[MAX_DW];
          load_wire(&f, p, io[r] + (size_t)next * work_elems + off_el, left);
          cell_send(&f, CELL(scat[next], r, slot, w), p, flag);
        }
      /* reduce own chunk with the peers' messages in order rank+1, rank+2, ... (l.130-171),
       * gather-push (l.173-177), store (l.181-186) */
      for (int r = 0; r < N && rc == 0; ++r) {
        uint32_t v[MAX_DW];
        load_wire(&f, v, io[r] + (size_t)r * work_elems + off_el, left);
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          uint32_t m[MAX_DW];
          if (cell_recv(&f, CELL(scat[r], next, slot, w), m, flag)) { rc = -1; break; }
          accum(v, m, f.cap_dw);
        }
        if (rc) break;
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          cell_send(&f, CELL(gath[next], r, slot, w), v, flag);
        }
        store_wire(&f, io[r] + (size_t)r * work_elems + off_el, v, left);
      }
      /* collect the other chunks (l.190-206) */
      for (int r = 0; r < N && rc == 0; ++r)
        for (int i = 0; i < N - 1; ++i) {
          const int next = (r + i + 1) % N;
          uint32_t m[MAX_DW];
          if (cell_recv(&f, CELL(gath[r], next, slot, w), m, flag)) { rc = -1; break; }
          store_wire(&f, io[r] + (size_t)next * work_elems + off_el, m, left);
        }
    }
  }
  for (int r = 0; r < N; ++r) {
    free(scat[r]);
    free(gath[r]);
  }
  return rc;
}

/* AllGather<T,N,Proto,RingTransmit,16> (allgather.hpp:79-100 + sequential_transmit.hpp:
 * 474-516, 396-428): the whole input is one work item list (workSize = bytes of one
 * input); rank r stores its own slice, sends it on, forwards N-2 slices and stores the
 * last.  out[r] holds N * n halves; out[r] + r * n may be in[r] itself (l.496-497). */
int vro_emulate_allgather_ring(uint16_t *const out[], const uint16_t *const in[], int nranks, size_t n,
                               int wire_kind, int groups, int subgroups, uint32_t seq_no) {
  const int N = nranks;
  if (N < 2 || N > MAXR || (N & (N - 1))) return -2;          /* uint32 wrap needs 2^k */
  const wire_fmt f = make_fmt(wire_kind);
  const size_t W = (size_t)groups * (size_t)subgroups;
  if (W == 0 || W > MAXLAUNCH) return -3;
  const size_t work_elems = n, work_bytes = n * 2;
  const size_t cap = (size_t)f.cap_dw * 4;
  const size_t loop = W * cap;
  enum { NSLOT = 4 };
  const size_t cells = (size_t)N * NSLOT * W;
  cell *gath[MAXR];
  for (int r = 0; r < N; ++r) gath[r] = calloc(cells, sizeof(cell));
  int rc = 0;
  size_t t = 0;
  for (size_t goff = 0; goff < work_bytes && rc == 0; goff += loop, ++t) {
    const uint32_t flag = seq_no + (uint32_t)(t / NSLOT);
    const size_t slot = (seq_no + t) % NSLOT;
    for (size_t w = 0; w < W && rc == 0; ++w) {
      const size_t wire_off = w * cap + goff;
      if (wire_off >= work_bytes) continue;
      const size_t off_el = wire_off / 2, left = work_elems - off_el;
      /* own slice: store unless the input already is the output slot, send on */
      for (int r = 0; r < N; ++r) {
        const int peer = r, next = (r + 1) % N;
        uint32_t p[MAX_DW];
        load_wire(&f, p, in[r] + off_el, left);
        cell_send(&f, CELL(gath[next], peer, slot, w), p, flag);
        uint16_t *o = out[r] + (size_t)peer * work_elems + off_el;
        if (o != in[r] + off_el) store_wire(&f, o, p, left);
      }
      /* p_idx = -1, -2, ...: receive slice (rank - i), forward it except on the last hop */
      for (int i = 1; i < N && rc == 0; ++i)
        for (int r = 0; r < N; ++r) {
          const int peer = (r + N - i) % N, next = (r + 1) % N;
          uint32_t m[MAX_DW];
          if (cell_recv(&f, CELL(gath[r], peer, slot, w), m, flag)) { rc = -1; break; }
          if (i < N - 1) cell_send(&f, CELL(gath[next], peer, slot, w), m, flag);
          store_wire(&f, out[r] + (size_t)peer * work_elems + off_el, m, left);
        }
    }
  }
#undef CELL
  for (int r = 0; r < N; ++r) free(gath[r]);
  return rc;
}

int vro_emulate_bisect(uint16_t *const io[], int nranks, size_t n, int groups, int subgroups,
                       uint32_t seq_no) {
  const int N = nranks, B = nranks / 2;
  if (N < 4 || N > MAXR || (N & 1) || n % (size_t)N) return -2;
  const wire_fmt f = make_fmt(VRO_WIRE_RT64_128);
  const size_t W = (size_t)groups * (size_t)subgroups;
  if (W < (size_t)B || W % (size_t)B || W > MAXLAUNCH) return -3;
  const size_t work_elems = n / (size_t)N, work_bytes = work_elems * 2;
  const size_t cap = 120, cols = W / (size_t)B, loop = cols * cap;
  const size_t ring_dw = (size_t)NSLOT_PAR * MSG_DW;
  const size_t far_base = (size_t)MAXLAUNCH * ring_dw;        /* ringSize*maxLaunch      */
  const size_t buf_dw = far_base + (W + (size_t)B) * ring_dw;
  uint32_t *scat[MAXR], *gath[MAXR];
  for (int r = 0; r < N; ++r) {
    scat[r] = calloc(buf_dw, 4);
    gath[r] = calloc(buf_dw, 4);
  }
  uint32_t(*regs)[MAX_DW] = malloc(sizeof(uint32_t[MAX_DW]) * (size_t)N * (size_t)B);
  int rc = 0;
  size_t t = 0;
  /* Element offset of rank r's close / far half (bisect_transmit.hpp:439-444). */
#define CLOSE_OFF(r) (((r)&1) ? work_elems * (size_t)B : 0)
#define FAR_OFF(r) (((r)&1) ? 0 : work_elems * (size_t)B)
  for (size_t goff = 0; goff < work_bytes && rc == 0; goff += loop, ++t) {
    const uint32_t flag = seq_no + (uint32_t)(t / NSLOT_PAR);
    const size_t slot = t % NSLOT_PAR;
    for (size_t x = 0; x < cols && rc == 0; ++x) {
      const size_t wire_off = x * cap + goff;
      if (wire_off >= work_bytes) continue;
      const size_t off_el = wire_off / 2, left = work_elems - off_el;
      const size_t wg = x * (size_t)B;                        /* wireId_g                */
      uint32_t msg[32], tmp[MAX_DW];
      /* scatterFar: send the half this rank does not own to the pair rank. */
      for (int r = 0; r < N; ++r)
        for (int y = 0; y < B; ++y) {
          load_wire(&f, tmp, io[r] + FAR_OFF(r) + (size_t)y * work_elems + off_el, left);
          pack_msg(&f, msg, tmp, flag);
          memcpy(scat[r ^ 1] + far_base + (wg + (size_t)y) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
        }
      /* close part: pair sum, then scatter to the same-parity owner. */
      for (int r = 0; r < N && rc == 0; ++r)
        for (int y = 0; y < B; ++y) {
          uint32_t *v = regs[r * B + y];
          load_wire(&f, v, io[r] + CLOSE_OFF(r) + (size_t)y * work_elems + off_el, left);
          if (unpack_msg(&f, scat[r] + far_base + (wg + (size_t)y) * ring_dw + slot * MSG_DW, tmp, flag)) {
            rc = -1;
            break;
          }
          accum(v, tmp, f.cap_dw);
          if (y != r / 2) {
            pack_msg(&f, msg, v, flag);
            const int owner = 2 * y + (r & 1);
            memcpy(scat[owner] + (wg + (size_t)(r / 2)) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
          }
        }
      /* owners: add the other pair sums in order l+1, l+2, ...; gather-push. */
      for (int r = 0; r < N && rc == 0; ++r) {
        const int l = r / 2;
        uint32_t *v = regs[r * B + l];
        for (int i = 0; i < B - 1; ++i) {
          const int l_next = (l + i + 1) % B;
          if (unpack_msg(&f, scat[r] + (wg + (size_t)l_next) * ring_dw + slot * MSG_DW, tmp, flag)) {
            rc = -1;
            break;
          }
          accum(v, tmp, f.cap_dw);
        }
        pack_msg(&f, msg, v, flag);
        for (int i = 0; i < B - 1; ++i) {
          const int next = (r + i * 2 + 2) % N;
          memcpy(gath[next] + (wg + (size_t)l) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
        }
      }
      /* non-owners receive the gathered result; everyone forwards to the pair and stores. */
      for (int r = 0; r < N && rc == 0; ++r)
        for (int y = 0; y < B; ++y) {
          uint32_t *v = regs[r * B + y];
          if (y != r / 2 &&
              unpack_msg(&f, gath[r] + (wg + (size_t)y) * ring_dw + slot * MSG_DW, v, flag)) {
            rc = -1;
            break;
          }
          pack_msg(&f, msg, v, flag);
          memcpy(gath[r ^ 1] + far_base + (wg + (size_t)y) * ring_dw + slot * MSG_DW, msg, MSG_BYTES);
          store_wire(&f, io[r] + CLOSE_OFF(r) + (size_t)y * work_elems + off_el, v, left);
        }
      /* pollFarGatherOutput: store the other half from the pair's forward. */
      for (int r = 0; r < N && rc == 0; ++r)
        for (int y = 0; y < B; ++y) {
          if (unpack_msg(&f, gath[r] + far_base + (wg + (size_t)y) * ring_dw + slot * MSG_DW, tmp, flag)) {
            rc = -1;
            break;
          }
          store_wire(&f, io[r] + FAR_OFF(r) + (size_t)y * work_elems + off_el, tmp, left);
        }
    }
  }
#undef CLOSE_OFF
#undef FAR_OFF
  for (int r = 0; r < N; ++r) {
    free(scat[r]);
    free(gath[r]);
  }
  free(regs);
  return rc;
}

int vro_emulate_parallel_dt(int dtype, uint16_t *const io[], int nranks, size_t n, int wire, int groups,
                            int subgroups, uint32_t seq_no) {
  g_emul_dtype = dtype;
  const int rc = vro_emulate_parallel(io, nranks, n, wire, groups, subgroups, seq_no);
  g_emul_dtype = VRO_F16;
  return rc;
}

int vro_emulate_bisect_dt(int dtype, uint16_t *const io[], int nranks, size_t n, int groups,
                          int subgroups, uint32_t seq_no) {
  g_emul_dtype = dtype;
  const int rc = vro_emulate_bisect(io, nranks, n, groups, subgroups, seq_no);
  g_emul_dtype = VRO_F16;
  return rc;
}
