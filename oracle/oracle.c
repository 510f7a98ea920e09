/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the arithmetic and index math of Fairring's K-way
 * gradient-slice reduction. Only tests, the smoke check and the benchmark's
 * CPU-baseline leg may link or call this file; the shipped library never does.
 *
 * What each function follows in the reference tree (paths relative to it):
 *   orc_sum_f32 / orc_sum_bf16 / orc_max_*  -> fairring/device.cc:108-131
 *       (doReduction: result = reduce over dim 0 of operand[K, n]); the order
 *       of additions is the sequential at::add chain acc = x[0];
 *       acc = acc + x[k] for k = 1..K-1, which is the contract this build is
 *       held to (the reference delegates the arithmetic to ATen).
 *   orc_compute_layout                       -> fairring/utils.h:288-327
 *   orc_ceil_of_ratio / round helpers        -> fairring/utils.h:258-274
 *   orc_num_slices / orc_slice_bounds        -> fairring/device.cc:315-326
 *   orc_readme_layout                        -> README.md:61-62 (the
 *       FAIRRING_TOTAL_MEMORY / FAIRRING_SLICE_SIZE pair)
 *
 *   orc_compressed_sum and the PRE_MUL / PRE_DIV scale modes follow torch's DDP
 *       hooks on either side of the allreduce the reference serves
 *       (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:18-93);
 *       pinned against those very expressions run by the installed torch.
 *
 * Pinned by (see tests/test_oracle.py): the installed ATen's add chain and
 * sum(dim=0) (K <= 17) bit for bit, ATen's bf16 sum over dim 0, an exact
 * rational-arithmetic brute force with explicit round-to-nearest-even on tiny
 * inputs, the all-ones and arange known answers of
 * benchmark/benchmark.cc:130-186, and hand-evaluated layout/slicing tables.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, optional OpenMP).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORC_SCALE_NONE 0 /* out = acc */
#define ORC_SCALE_MUL 1  /* out = acc * scale   (scale = 1/K, exact for K=2^p) */
#define ORC_SCALE_DIV 2  /* out = acc / scale   (scale = K, at::div semantics) */
/* Pre-scale: every contribution is scaled, and rounded to its storage type,
 * before the fold; what DDP does to each rank's bucket ahead of the
 * allreduce (tensor.div_(world) in torch's allreduce_hook). */
#define ORC_SCALE_PRE_MUL 3 /* term = x[k] * scale */
#define ORC_SCALE_PRE_DIV 4 /* term = x[k] / scale */

static inline float apply_scale(float acc, int mode, float scale) {
  if (mode == ORC_SCALE_MUL) return acc * scale;
  if (mode == ORC_SCALE_DIV) return acc / scale;
  return acc;
}

static inline float pre_scale(float x, int mode, float scale) {
  if (mode == ORC_SCALE_PRE_MUL) return x * scale;
  if (mode == ORC_SCALE_PRE_DIV) return x / scale;
  return x;
}

/* fp32: left fold in contribution order starting from x[0] (not from 0). */
void orc_sum_f32(float* out, const float* const* in, int K, int64_t n,
                 int scale_mode, float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float acc = pre_scale(in[0][i], scale_mode, scale);
    for (int k = 1; k < K; ++k) acc = acc + pre_scale(in[k][i], scale_mode, scale);
    out[i] = apply_scale(acc, scale_mode, scale);
  }
}

/* Same chain, blocked over contributions the way a streaming CPU
 * implementation would run it (acc = x0; acc += xk ...), used as the timed
 * CPU baseline. Bit-identical to orc_sum_f32. */
void orc_sum_f32_chain(float* out, const float* const* in, int K, int64_t n,
                       int scale_mode, float scale) {
#pragma omp parallel
  {
    const int64_t B = 4096;
#pragma omp for schedule(static)
    for (int64_t b = 0; b < (n + B - 1) / B; ++b) {
      int64_t lo = b * B, hi = lo + B < n ? lo + B : n;
      for (int64_t i = lo; i < hi; ++i) out[i] = pre_scale(in[0][i], scale_mode, scale);
      for (int k = 1; k < K; ++k)
        for (int64_t i = lo; i < hi; ++i)
          out[i] = out[i] + pre_scale(in[k][i], scale_mode, scale);
      if (scale_mode == ORC_SCALE_MUL || scale_mode == ORC_SCALE_DIV)
        for (int64_t i = lo; i < hi; ++i)
          out[i] = apply_scale(out[i], scale_mode, scale);
    }
  }
}

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* Round-to-nearest-even fp32 -> bf16, NaN -> 0x7FC0. */
static inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)((u + bias) >> 16);
}

/* bf16 storage: exact upcast, fp32 accumulation in contribution order, scale
 * in fp32, one rounding on store. */
void orc_sum_bf16(uint16_t* out, const uint16_t* const* in, int K, int64_t n,
                  int scale_mode, float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const int pre = scale_mode >= ORC_SCALE_PRE_MUL;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
      float t = bf16_to_f32(in[k][i]);
      /* a pre-scaled term is a bf16 tensor of its own: rounded before the fold */
      if (pre) t = bf16_to_f32(f32_to_bf16_rne(pre_scale(t, scale_mode, scale)));
      acc = k == 0 ? t : acc + t;
    }
    out[i] = f32_to_bf16_rne(apply_scale(acc, scale_mode, scale));
  }
}

/* MAX with NaN propagation (ATen amax): any NaN in a lane gives NaN. */
static inline float max_nan(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  return a > b ? a : b;
}

void orc_max_f32(float* out, const float* const* in, int K, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float acc = in[0][i];
    for (int k = 1; k < K; ++k) acc = max_nan(acc, in[k][i]);
    out[i] = acc;
  }
}

void orc_max_bf16(uint16_t* out, const uint16_t* const* in, int K, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float acc = bf16_to_f32(in[0][i]);
    for (int k = 1; k < K; ++k) acc = max_nan(acc, bf16_to_f32(in[k][i]));
    out[i] = f32_to_bf16_rne(acc);
  }
}

/* ---- integer helpers -------------------------------------------------- */

int64_t orc_ceil_of_ratio(int64_t num, int64_t den) {
  if (num == 0) return 0;
  return (num - 1) / den + 1;
}

int64_t orc_round_down(int64_t val, int64_t factor) {
  return (val / factor) * factor;
}

int64_t orc_round_up(int64_t val, int64_t factor) {
  return orc_ceil_of_ratio(val, factor) * factor;
}

#define ORC_ALIGNMENT 8

/* out4 = {slotSizeInBytes, sliceSizeInBytes, numPaddingSlots, numStagingSlots}.
 * Returns 0, or 1/2 where the reference terminates (first/second check). */
int orc_compute_layout(int64_t max_mem, int64_t max_pad, int64_t min_par,
                       int64_t num_machines, int64_t devs_per_machine,
                       int64_t* out4) {
  int64_t one_pad = devs_per_machine * num_machines * ORC_ALIGNMENT;
  int64_t num_pad_slots = max_pad / one_pad;
  if (!(min_par <= num_pad_slots)) return 1;
  int64_t slice = INT64_MAX, slot = 0, num_staging = 0;
  if (devs_per_machine == 1) {
    int64_t pad_mem = 2 * min_par * devs_per_machine * num_machines * ORC_ALIGNMENT;
    if (!(pad_mem <= max_mem)) return 2;
    slot = orc_round_down((max_mem - pad_mem) / min_par,
                          devs_per_machine * num_machines * ORC_ALIGNMENT);
    slice = slot * devs_per_machine;
    num_staging = min_par;
    num_pad_slots = min_par;
  }
  out4[0] = slot;
  out4[1] = slice;
  out4[2] = num_pad_slots;
  out4[3] = num_staging;
  return 0;
}

/* README regime: number of staging slots that TOTAL_MEMORY holds. */
int64_t orc_readme_layout(int64_t total_memory, int64_t slice_size) {
  return total_memory / slice_size;
}

int64_t orc_num_slices(int64_t numel, int64_t slice_bytes, int64_t elsize) {
  int64_t max_elems = slice_bytes / elsize;
  return orc_ceil_of_ratio(numel, max_elems);
}

/* bounds2 = {offsetInElems, sliceSizeInElems} of slice idx. */
void orc_slice_bounds(int64_t numel, int64_t slice_bytes, int64_t elsize,
                      int64_t idx, int64_t* bounds2) {
  int64_t max_elems = slice_bytes / elsize;
  int64_t off = idx * max_elems;
  int64_t rem = numel - off;
  bounds2[0] = off;
  bounds2[1] = max_elems < rem ? max_elems : rem;
}

/* ---- thread control for the timed baseline ----------------------------- */
#ifdef _OPENMP
#include <omp.h>
void orc_set_threads(int n) { omp_set_num_threads(n); }
int orc_max_threads(void) { return omp_get_max_threads(); }
#else
void orc_set_threads(int n) { (void)n; }
int orc_max_threads(void) { return 1; }
#endif

/* ---- the other element types the reference maps to NCCL types ------------
 * (fairring/utils.h:221-245): fp16 folds in fp32 with one rounding on the
 * store (ATen's accumulate type for Half), fp64 in fp64, integers with
 * two's-complement wrap-around in their own width. Same left fold. */

/* IEEE binary16 <-> binary32 without relying on compiler half support. */
static inline float f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_f16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu)); /* NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536 (incl. inf) -> inf */
  if (a >= 0x38800000u) { /* normal half range */
    uint32_t m = a - 0x38000000u; /* rebias exponent by 112 */
    uint32_t r = m >> 13;
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r; /* may carry into inf: correct */
    return (uint16_t)(sign | r);
  }
  if (a < 0x33000000u) return (uint16_t)sign; /* < 2^-25: rounds to zero */
  /* subnormal half: value = mant * 2^(e-150), target unit 2^-24 */
  uint32_t e = a >> 23;
  uint32_t mant = (a & 0x7FFFFFu) | 0x800000u;
  uint32_t shift = 126 - e; /* e in [102, 112] -> shift in [14, 24] */
  uint32_t r = mant >> shift;
  uint32_t rem = mant & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (r & 1u))) ++r;
  return (uint16_t)(sign | r);
}

void orc_sum_f16(uint16_t* out, const uint16_t* const* in, int K, int64_t n, int scale_mode,
                 float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const int pre = scale_mode >= ORC_SCALE_PRE_MUL;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
      float t = f16_to_f32(in[k][i]);
      if (pre) t = f16_to_f32(f32_to_f16_rne(pre_scale(t, scale_mode, scale)));
      acc = k == 0 ? t : acc + t;
    }
    out[i] = f32_to_f16_rne(apply_scale(acc, scale_mode, scale));
  }
}

void orc_max_f16(uint16_t* out, const uint16_t* const* in, int K, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float acc = f16_to_f32(in[0][i]);
    for (int k = 1; k < K; ++k) acc = max_nan(acc, f16_to_f32(in[k][i]));
    out[i] = f32_to_f16_rne(acc);
  }
}

void orc_sum_f64(double* out, const double* const* in, int K, int64_t n, int scale_mode,
                 float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    double acc = 0.0;
    for (int k = 0; k < K; ++k) {
      double t = in[k][i];
      if (scale_mode == ORC_SCALE_PRE_MUL) t = t * (double)scale;
      if (scale_mode == ORC_SCALE_PRE_DIV) t = t / (double)scale;
      acc = k == 0 ? t : acc + t;
    }
    if (scale_mode == ORC_SCALE_MUL) acc = acc * (double)scale;
    if (scale_mode == ORC_SCALE_DIV) acc = acc / (double)scale;
    out[i] = acc;
  }
}

void orc_max_f64(double* out, const double* const* in, int K, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    double acc = in[0][i];
    for (int k = 1; k < K; ++k) {
      double b = in[k][i];
      acc = (acc != acc) ? acc : ((b != b) ? b : (acc > b ? acc : b));
    }
    out[i] = acc;
  }
}

#define ORC_INT_REDUCE(NAME, T, UT)                                               \
  void orc_sum_##NAME(T* out, const T* const* in, int K, int64_t n) {              \
    for (int64_t i = 0; i < n; ++i) {                                              \
      UT acc = (UT)in[0][i];                                                       \
      for (int k = 1; k < K; ++k) acc = (UT)(acc + (UT)in[k][i]);                  \
      out[i] = (T)acc;                                                             \
    }                                                                              \
  }                                                                                \
  void orc_max_##NAME(T* out, const T* const* in, int K, int64_t n) {              \
    for (int64_t i = 0; i < n; ++i) {                                              \
      T acc = in[0][i];                                                            \
      for (int k = 1; k < K; ++k) acc = in[k][i] > acc ? in[k][i] : acc;           \
      out[i] = acc;                                                                \
    }                                                                              \
  }

ORC_INT_REDUCE(i32, int32_t, uint32_t)
ORC_INT_REDUCE(i64, int64_t, uint64_t)
ORC_INT_REDUCE(u8, uint8_t, uint8_t)
ORC_INT_REDUCE(i8, int8_t, uint8_t)

/* ---- gradient compression around the reduction ---------------------------
 * What torch's bf16/fp16 compress hooks do on every rank on either side of the
 * allreduce that fairring/process_group.cc:131-155 serves
 * (torch:distributed/algorithms/ddp_comm_hooks/default_hooks.py:57-93):
 *   compressed = buffer.to(wire).div_(world)      -- two roundings to wire
 *   allreduce(compressed)                         -- fp32 fold, one rounding
 *   buffer.copy_(result)                          -- exact widening
 * Contribution raw_index (if >= 0) is this rank's fp32 buffer and goes through
 * the compress step here; the others are peers' tensors, already in the wire
 * type. scale_mode MUL computes x * scale (ATen on the GPU multiplies by the
 * reciprocal of a scalar divisor), DIV computes x / scale (ATen on the CPU).
 * wire: 0 = bf16, 1 = fp16. out_f32: store the result widened to fp32. */
static inline float wire_to_f32(uint16_t w, int wire) {
  return wire ? f16_to_f32(w) : bf16_to_f32(w);
}

static inline uint16_t f32_to_wire(float f, int wire) {
  return wire ? f32_to_f16_rne(f) : f32_to_bf16_rne(f);
}

void orc_compressed_sum(void* out, int out_f32, const void* const* in, int K, int raw_index,
                        int64_t n, int wire, int scale_mode, float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
      float t;
      if (k == raw_index) {
        const float x = ((const float*)in[k])[i];
        const float cast = wire_to_f32(f32_to_wire(x, wire), wire);
        t = wire_to_f32(f32_to_wire(apply_scale(cast, scale_mode, scale), wire), wire);
      } else {
        t = wire_to_f32(((const uint16_t*)in[k])[i], wire);
      }
      acc = k == 0 ? t : acc + t;
    }
    const uint16_t r = f32_to_wire(acc, wire);
    if (out_f32) {
      ((float*)out)[i] = wire_to_f32(r, wire);
    } else {
      ((uint16_t*)out)[i] = r;
    }
  }
}
