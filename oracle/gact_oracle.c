/*
 * CPU restatement of GACT's saved-activation compression arithmetic.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the timed CPU baseline; nothing in the shipped library
 * links, loads or calls it.
 *
 * Each function follows the reference source it cites (paths relative to the
 * reference checkout).  Compile with -ffp-contract=off: every floating-point
 * operation below is meant literally, and the one fused multiply-add of the
 * path is spelled fmaf().
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   minimax        pinned   against numpy min/max (the reference's own tests
 *                           compare with torch.min/max)
 *   scale          pinned   closed form in exact rational arithmetic
 *   pack / unpack  pinned   exact rational (fractions.Fraction) brute force,
 *                           code invariants, hand-built layout cases, the
 *                           reference's one-hot round trips
 *   philox4x32 (10 and 7 rounds)  pinned   Random123 known-answer vectors
 *   reference noise stream (cuRAND Philox state walk + uniform map):
 *                  the reference holds no vector for it and cuRAND is not in
 *                  this image; restated from its published header semantics
 *                  and pinned on the GPU against hipRAND's cuRAND-compatible
 *                  Philox as torch's device generator draws it (seed, subsequence,
 *                  offset -> key / counter, word order, next block, uniform map:
 *                  tests/test_gpu_philox_library.py).  PARITY UNPINNED only in
 *                  that cuRAND itself was never run
 *   fast noise stream        our own definition, no reference counterpart
 *   calc_precision pinned   against the reference's calc_precision.cc compiled
 *                           as-is into oracle/_ref (when built) + hand cases
 *   mask pack/unpack pinned round trip identity + index formula
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__F16C__)
#include <immintrin.h>
#endif

#define GACT_F32 0
#define GACT_F16 1

/* ------------------------------------------------------------------------- */
/* IEEE binary16 <-> binary32, round-to-nearest-even (what c10::Half does).  */
/* ------------------------------------------------------------------------- */
static inline float half_bits_to_float_sw(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline uint16_t float_to_half_bits_sw(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* < 2^-25 (or == 2^-25, tie to even 0) */
    return sign;
  }
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                 /* bits to drop */
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
  uint32_t out;
  if (hexp == 0) {
    out = kept; /* may carry into exponent 1: correct encoding */
  } else {
    out = ((hexp - 1) << 10) + kept; /* kept includes the hidden bit (0x400) */
  }
  return (uint16_t)(sign | out);
}

static inline float h2f(uint16_t h) {
#if defined(__F16C__)
  return _cvtsh_ss(h);
#else
  return half_bits_to_float_sw(h);
#endif
}
static inline uint16_t f2h(float f) {
#if defined(__F16C__)
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
  return float_to_half_bits_sw(f);
#endif
}

/* exported so the tests can pin both converters against numpy */
float gact_oracle_h2f_sw(uint16_t h) { return half_bits_to_float_sw(h); }
uint16_t gact_oracle_f2h_sw(float f) { return float_to_half_bits_sw(f); }
float gact_oracle_h2f(uint16_t h) { return h2f(h); }
uint16_t gact_oracle_f2h(float f) { return f2h(f); }

/* round a float through half and back: the value a c10::Half holds */
static inline float rh(float f) { return h2f(f2h(f)); }

/* ------------------------------------------------------------------------- */
/* P1  per-row min / max.                                                    */
/* gact/gact/cpp_extension/minimax_cuda_kernel.cu:23-67: accumulators start  */
/* at +-1e30 (narrowed to the tensor type, so +-inf in half), updated with   */
/* std::min / std::max, which keep the accumulator when the comparison with  */
/* a NaN is false.  The order of the comparisons does not change the value.  */
/* ------------------------------------------------------------------------- */
void gact_oracle_minimax(const void* data, int dtype, int64_t N, int64_t D, void* mn, void* mx) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    if (dtype == GACT_F32) {
      const float* x = (const float*)data + n * D;
      float lo = 1e30f, hi = -1e30f;
      for (int64_t d = 0; d < D; d++) {
        float v = x[d];
        lo = (v < lo) ? v : lo;
        hi = (hi < v) ? v : hi;
      }
      ((float*)mn)[n] = lo;
      ((float*)mx)[n] = hi;
    } else {
      const uint16_t* x = (const uint16_t*)data + n * D;
      float lo = rh(1e30f), hi = rh(-1e30f); /* +inf, -inf */
      uint16_t lob = f2h(1e30f), hib = f2h(-1e30f);
      for (int64_t d = 0; d < D; d++) {
        float v = h2f(x[d]);
        if (v < lo) { lo = v; lob = x[d]; }
        if (hi < v) { hi = v; hib = x[d]; }
      }
      ((uint16_t*)mn)[n] = lob;
      ((uint16_t*)mx)[n] = hib;
    }
  }
}

/* ------------------------------------------------------------------------- */
/* P2  scale = T(2^b - 1) / (max - min + 2e-6).                              */
/* quantization_cuda_kernel.cu:23-35.  `max - min` is an operation of the    */
/* tensor type T (so it is rounded to half for half tensors); 2e-6 is a      */
/* double literal, which promotes the sum and the quotient to double; the    */
/* store narrows double -> T (through float for half: c10::Half has only a   */
/* float constructor).                                                       */
/* ------------------------------------------------------------------------- */
static inline float scale_f32(float mn, float mx, int bits) {
  float range = mx - mn;
  double q = (double)(float)((1 << bits) - 1) / ((double)range + 2e-6);
  return (float)q;
}
static inline uint16_t scale_f16(uint16_t mn, uint16_t mx, int bits) {
  float range = rh(h2f(mx) - h2f(mn));
  double q = (double)rh((float)((1 << bits) - 1)) / ((double)range + 2e-6);
  return f2h((float)q);
}

void gact_oracle_scale(const void* mn, const void* mx, int dtype, int bits, int64_t count, void* scale) {
  for (int64_t i = 0; i < count; i++) {
    if (dtype == GACT_F32)
      ((float*)scale)[i] = scale_f32(((const float*)mn)[i], ((const float*)mx)[i], bits);
    else
      ((uint16_t*)scale)[i] = scale_f16(((const uint16_t*)mn)[i], ((const uint16_t*)mx)[i], bits);
  }
}

/* ------------------------------------------------------------------------- */
/* Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2,  */
/* 3", SC'11; Random123).  This is the generator behind cuRAND's             */
/* curandStatePhilox4_32_10_t, which the reference instantiates at           */
/* quantization_cuda_kernel.cu:55-56.                                        */
/* ------------------------------------------------------------------------- */
void gact_oracle_philox4x32(const uint32_t ctr[4], const uint32_t key[2], int rounds, uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < rounds; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
void gact_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  gact_oracle_philox4x32(ctr, key, 10, out);
}

/* cuRAND's curand_uniform(): x * 2^-32 + 2^-33 evaluated in float, so the   */
/* result lies in (0, 1] (x = 2^32-1 converts to 2^32 and gives exactly 1).  */
float gact_oracle_curand_uniform(uint32_t x) {
  float xf = (float)x;                         /* round to nearest even */
  return xf * 2.3283064365386963e-10f + 1.1641532182693481e-10f; /* one rounding: the product is exact */
}

/* The reference noise stream.  quantization_cuda_kernel.cu:106-114 builds a  */
/* fresh generator, seeds it and takes (seed, offset 0); :55-56 initialises   */
/* one Philox state per output byte with curand_init(seed, subsequence =      */
/* byte index, offset); :65 draws one uniform per field in field order.       */
/* cuRAND's state walk: key = seed (lo, hi); counter = (offset/4 lo, hi,      */
/* subsequence lo, hi); draws consume the block's words x, y, z, w and then   */
/* the 128-bit counter is incremented by one.                                 */
static inline float ref_stream_uniform(uint64_t seed, uint64_t byte_index, int draw) {
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t ctr[4] = {(uint32_t)(draw >> 2), 0u, (uint32_t)byte_index, (uint32_t)(byte_index >> 32)};
  uint32_t out[4];
  gact_oracle_philox4x32_10(ctr, key, out);
  return gact_oracle_curand_uniform(out[draw & 3]);
}

/* The fast noise stream (ours; the reference has no counterpart).  Philox4x32 */
/* with seven rounds (the same round function; the fewest rounds for which    */
/* Random123's authors report that the generator passes BigCrush; its         */
/* kat_vectors hold the 7-round known answers too), key = seed.  Every 512    */
/* consecutive elements of the flattened tensor (two groups of 256) draw 16   */
/* blocks of 16 bytes.  Element E, with column d = E%256 and d' = d%128:      */
/* block (E/512)*16 + d'/8 (counter = (0, 0, block lo, block hi)), of its 16  */
/* output bytes (word by word, low byte first) byte ((E/256)%2)*8 + d'%8, h.   */
/* The draw is centred: c = (2h - 255)/512, i.e. (h + 0.5)/256 - 1/2, one of  */
/* 256 values symmetric about 0, strictly inside (-1/2, 1/2); for d >= 128    */
/* the element takes -c: the two elements half a group apart share one draw,  */
/* mirrored (an antithetic pair: both uniform on the same grid; covariance of */
/* their rounding errors <= 0).  The code is rint(max(y, 0)) with the noise   */
/* added where the reference adds its own: y = fma(x - min, scale, c) for      */
/* float, float(half product) + c for half - the reference's                   */
/* (.. + u) - 0.5 with u = c + 1/2, rounded once instead of twice.             */
#define GACT_FAST_ROUNDS 7
static inline uint64_t fast_stream_block(uint64_t elem) { return (elem >> 9) * 16u + ((elem & 127u) >> 3); }
static inline int fast_stream_byte(uint64_t elem) { return (int)(((elem >> 8) & 1u) * 8u + (elem & 7u)); }
static inline float fast_stream_centred_from_block(const uint32_t out[4], uint64_t elem) {
  int b = fast_stream_byte(elem);
  uint32_t h = (out[b >> 2] >> (8 * (b & 3))) & 0xffu;
  float c = (float)(2 * (int32_t)h - 255) * 0.001953125f; /* (2h - 255) * 2^-9, exact */
  return (elem & 128u) ? -c : c;
}
static inline float fast_stream_centred(uint64_t seed, uint64_t elem) {
  uint64_t blk = fast_stream_block(elem);
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t ctr[4] = {0u, 0u, (uint32_t)blk, (uint32_t)(blk >> 32)};
  uint32_t out[4];
  gact_oracle_philox4x32(ctr, key, GACT_FAST_ROUNDS, out);
  return fast_stream_centred_from_block(out, elem);
}
/* the same draw as a uniform on (0, 1): c + 1/2 = (2h + 1)/512, exact */
static inline float fast_stream_uniform(uint64_t seed, uint64_t elem) { return fast_stream_centred(seed, elem) + 0.5f; }

#define GACT_NOISE_CONST 0  /* u = 0.5 for every element: deterministic rounding */
#define GACT_NOISE_INJECT 1 /* u read from a float tensor shaped like the data  */
#define GACT_NOISE_REF 2    /* the reference's cuRAND-compatible stream         */
#define GACT_NOISE_FAST 3   /* one 7-round Philox block per 32 elements, 8-bit centred noise */

/* Materialise the noise tensor a given mode uses, in data layout [N,G,D].    */
void gact_oracle_noise(int noise_mode, uint64_t seed, int bits, int64_t N, int64_t G, int64_t D, float* u) {
  const int wpt = 8 / bits;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    int64_t no = n / wpt;
    int ni = (int)(n % wpt);
    for (int64_t g = 0; g < G; g++)
      for (int64_t d = 0; d < D; d++) {
        int64_t id = (n * G + g) * D + d;
        int64_t byte_index = (no * G + g) * D + d;
        float v = 0.5f;
        if (noise_mode == GACT_NOISE_REF) v = ref_stream_uniform(seed, (uint64_t)byte_index, ni);
        else if (noise_mode == GACT_NOISE_FAST) v = fast_stream_uniform(seed, (uint64_t)id);
        u[id] = v;
      }
  }
}

/* ------------------------------------------------------------------------- */
/* P3  one quantisation code.                                                */
/* quantization_cuda_kernel.cu:66:                                           */
/*   val = __float2int_rn(fmax((data - min) * scale + noise - 0.5, 0.0f))    */
/* with `fmax` the macro of :14 ((a) > (b) ? (a) : (b)).                     */
/* float tensors: data-min is a float subtraction; the product and the       */
/* addition of the float noise are one expression, which both nvcc           */
/* (-fmad=true, its default) and hipcc (-ffp-contract=fast, its default)     */
/* contract into a single fused multiply-add, so a build of the reference    */
/* computes fmaf(t, scale, noise).  half tensors: data-min and the product   */
/* are c10::Half operators (computed in float, rounded to half), so nothing  */
/* can fuse; half + float gives float.  `- 0.5` promotes to double and is    */
/* exact there; the macro compares in double; __float2int_rn takes a float,  */
/* so the double narrows (round to nearest) and is then rounded to the       */
/* nearest-even integer with saturation.  Narrowing the exact double         */
/* difference equals the float subtraction y - 0.5f, and narrowing commutes   */
/* with the max against zero, so the whole tail is float arithmetic.         */
/* A NaN compares false and yields 0.                                        */
/* ------------------------------------------------------------------------- */
static inline int32_t float2int_rn_sat(float z) {
  if (!(z == z)) return 0;
  if (z >= 2147483648.0f) return 2147483647;
  if (z <= -2147483648.0f) return (int32_t)0x80000000u;
  return (int32_t)rintf(z); /* default rounding mode: ties to even */
}
static inline int32_t code_f32(float x, float mn, float s, float u) {
  float t = x - mn;
  float y = fmaf(t, s, u);
  float z = y - 0.5f;
  z = (z > 0.0f) ? z : 0.0f;
  return float2int_rn_sat(z);
}
static inline int32_t code_f16(uint16_t x, uint16_t mn, uint16_t s, float u) {
  float t = rh(h2f(x) - h2f(mn));
  float p = rh(t * h2f(s));
  float y = p + u;
  float z = y - 0.5f;
  z = (z > 0.0f) ? z : 0.0f;
  return float2int_rn_sat(z);
}
/* The fast stream's form of the same code: the draw c is centred, so the      */
/* reference's "+ noise - 0.5" is one addition.                                 */
static inline int32_t code_f32_centred(float x, float mn, float s, float c) {
  float t = x - mn;
  float z = fmaf(t, s, c);
  z = (z > 0.0f) ? z : 0.0f;
  return float2int_rn_sat(z);
}
static inline int32_t code_f16_centred(uint16_t x, uint16_t mn, uint16_t s, float c) {
  float t = rh(h2f(x) - h2f(mn));
  float p = rh(t * h2f(s));
  float z = p + c;
  z = (z > 0.0f) ? z : 0.0f;
  return float2int_rn_sat(z);
}

/* P3/P4  pack.  quantization_cuda_kernel.cu:38-71 (kernel) and :74-146       */
/* (launcher).  Output byte j = (no*G + g)*D + d ORs, for ni < 8/bits with    */
/* n = no*(8/bits) + ni < N, the value (code << ni*bits) truncated to 8 bits  */
/* (the accumulator is a uint8_t, so an over-range code spills into the next  */
/* fields and loses what does not fit).  Bytes written: N_round*G*D*bits/8;   */
/* the reference allocates one more byte and never writes it.                 */
void gact_oracle_pack(const void* data, const void* mn, const void* scale, int dtype, int bits, int64_t N,
                      int64_t G, int64_t D, int noise_mode, uint64_t seed, const float* noise,
                      uint8_t* packed) {
  const int wpt = 8 / bits;
  const int64_t n_outer = (N + wpt - 1) / wpt;
#pragma omp parallel for schedule(static)
  for (int64_t no = 0; no < n_outer; no++) {
    for (int64_t g = 0; g < G; g++) {
      for (int64_t d0 = 0; d0 < D; d0 += 8) {
        for (int64_t d = d0; d < d0 + 8 && d < D; d++) {
          int64_t j = (no * G + g) * D + d;
          uint8_t byte = 0;
          for (int ni = 0; ni < wpt; ni++) {
            int64_t n = no * wpt + ni;
            if (n >= N) break;
            int64_t id = (n * G + g) * D + d;
            int64_t sid = n * G + g;
            float u = 0.5f;
            if (noise_mode == GACT_NOISE_INJECT) u = noise[id];
            else if (noise_mode == GACT_NOISE_REF) u = ref_stream_uniform(seed, (uint64_t)j, ni);
            else if (noise_mode == GACT_NOISE_FAST) u = fast_stream_centred(seed, (uint64_t)id);
            int32_t val;
            if (noise_mode == GACT_NOISE_FAST) {
              if (dtype == GACT_F32)
                val = code_f32_centred(((const float*)data)[id], ((const float*)mn)[sid], ((const float*)scale)[sid], u);
              else
                val = code_f16_centred(((const uint16_t*)data)[id], ((const uint16_t*)mn)[sid],
                                       ((const uint16_t*)scale)[sid], u);
            } else if (dtype == GACT_F32)
              val = code_f32(((const float*)data)[id], ((const float*)mn)[sid], ((const float*)scale)[sid], u);
            else
              val = code_f16(((const uint16_t*)data)[id], ((const uint16_t*)mn)[sid],
                             ((const uint16_t*)scale)[sid], u);
            byte |= (uint8_t)((uint32_t)val << (ni * bits));
          }
          packed[j] = byte;
        }
      }
    }
  }
}

/* P5  unpack.  quantization_cuda_kernel.cu:149-177:                          */
/*   out = (T)code / scale + min   - a true division and an addition, each    */
/* an operation of T (for half: computed in float and rounded to half).       */
void gact_oracle_unpack(const uint8_t* packed, int bits, const void* scale, const void* mn, int dtype,
                        int64_t N, int64_t G, int64_t D, void* out) {
  const int wpt = 8 / bits;
  const int mask = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    int64_t no = n / wpt;
    int ni = (int)(n % wpt);
    for (int64_t g = 0; g < G; g++) {
      int64_t sid = n * G + g;
      for (int64_t d = 0; d < D; d++) {
        int64_t j = (no * G + g) * D + d;
        int64_t id = (n * G + g) * D + d;
        int val = (packed[j] >> (ni * bits)) & mask;
        if (dtype == GACT_F32) {
          float q = (float)val / ((const float*)scale)[sid];
          ((float*)out)[id] = q + ((const float*)mn)[sid];
        } else {
          float q = rh((float)val / h2f(((const uint16_t*)scale)[sid]));
          ((uint16_t*)out)[id] = f2h(q + h2f(((const uint16_t*)mn)[sid]));
        }
      }
    }
  }
}

/* P6 + P7 restated end to end for group size 256 and one channel group, as   */
/* gact/gact/ops.py:11-32 and :34-47,61-69 drive the kernels: the flattened   */
/* tensor is zero-padded to whole groups, min/max per group, scale, pack.     */
/* `x_padded` must already hold N*256 elements (the caller pads).             */
void gact_oracle_quantize(const void* x_padded, int dtype, int64_t N, int bits, int noise_mode, uint64_t seed,
                          const float* noise, uint8_t* packed, void* scale, void* mn, void* mx) {
  gact_oracle_minimax(x_padded, dtype, N, 256, mn, mx);
  gact_oracle_scale(mn, mx, dtype, bits, N, scale);
  gact_oracle_pack(x_padded, mn, scale, dtype, bits, N, 1, 256, noise_mode, seed, noise, packed);
}

/* ------------------------------------------------------------------------- */
/* P8  greedy bit allocation.  calc_precision.cc:66-118.                      */
/* A max-heap of (float key, int64 index) pairs compared lexicographically;   */
/* the keys are computed in double and narrowed to float when the pair is     */
/* pushed.  Because the index makes every pair distinct the pop order is the  */
/* descending total order, whatever the heap's shape, so a scan for the       */
/* maximum restates it exactly.  b_sum only counts entries that start above   */
/* 1 bit (:96-101).  Popping an empty queue is undefined in the reference;    */
/* here the loop stops and -1 is returned.                                    */
/* ------------------------------------------------------------------------- */
static inline int next_bits(int b) { return b == 32 ? 8 : b == 8 ? 4 : b == 4 ? 2 : b == 2 ? 1 : 0; }
static inline double prec_obj(float C, int b) {
  int nb = next_bits(b);
  int coeff_2 = ((1 << nb) - 1) * ((1 << nb) - 1);
  if (b == 32) return -(double)C / coeff_2;
  int coeff_1 = ((1 << b) - 1) * ((1 << b) - 1);
  return C * (1.0 / coeff_1 - 1.0 / coeff_2);
}
static inline float prec_key(float C, int b, int64_t w) {
  int delta_b = b - next_bits(b);
  return (float)(prec_obj(C, b) / (double)(w * delta_b));
}
int gact_oracle_calc_precision(int32_t* b, const float* C, const int64_t* w, int64_t L, double target) {
  float* key = (float*)malloc(sizeof(float) * (size_t)(L > 0 ? L : 1));
  uint8_t* live = (uint8_t*)calloc((size_t)(L > 0 ? L : 1), 1);
  double b_sum = 0;
  for (int64_t i = 0; i < L; i++)
    if (b[i] > 1) {
      key[i] = prec_key(C[i], b[i], w[i]);
      live[i] = 1;
      b_sum += (double)(b[i] * w[i]);
    }
  int rc = 0;
  while (b_sum > target) {
    int64_t best = -1;
    for (int64_t i = 0; i < L; i++) {
      if (!live[i]) continue;
      if (best < 0 || key[best] < key[i] || (!(key[i] < key[best]) && i > best)) best = i;
    }
    if (best < 0) { rc = -1; break; }
    int nb = next_bits(b[best]);
    int delta_b = b[best] - nb;
    b[best] = nb;
    b_sum -= (double)(w[best] * delta_b);
    if (nb > 1) key[best] = prec_key(C[best], nb, w[best]);
    else live[best] = 0;
  }
  free(key);
  free(live);
  return rc;
}

/* ------------------------------------------------------------------------- */
/* M1  dropout-mask bit packing.  quantization_cuda_kernel.cu:228-252 and     */
/* :276-288: within each block of 512 elements, element e = k*16 + w sets bit */
/* k of word w.  The reference stores all 16 words of a partial last block    */
/* past the end of its ceil(n/32)-word output; here the partial last block is */
/* instead packed sequentially (element e -> word e/32, bit e%32), which fits */
/* the output length.  Any nonzero byte counts as 1 (the reference converts   */
/* to bool).                                                                  */
/* ------------------------------------------------------------------------- */
void gact_oracle_mask_pack(const uint8_t* data, int64_t n, int32_t* mask) {
  int64_t words = (n + 31) / 32;
  int64_t full = n / 512;
  memset(mask, 0, (size_t)words * 4);
  for (int64_t blk = 0; blk < full; blk++)
    for (int e = 0; e < 512; e++)
      if (data[blk * 512 + e]) mask[blk * 16 + (e % 16)] |= (int32_t)(1u << (e / 16));
  for (int64_t e = full * 512; e < n; e++)
    if (data[e]) mask[full * 16 + (e - full * 512) / 32] |= (int32_t)(1u << ((e - full * 512) % 32));
}
void gact_oracle_mask_unpack(const int32_t* mask, int64_t n, uint8_t* out) {
  int64_t full = n / 512;
  for (int64_t blk = 0; blk < full; blk++)
    for (int e = 0; e < 512; e++)
      out[blk * 512 + e] = (uint8_t)(((uint32_t)mask[blk * 16 + (e % 16)] >> (e / 16)) & 1u);
  for (int64_t e = full * 512; e < n; e++)
    out[e] = (uint8_t)(((uint32_t)mask[full * 16 + (e - full * 512) / 32] >> ((e - full * 512) % 32)) & 1u);
}

/* threads the OpenMP loops above use (reported next to the CPU baseline figure) */
#ifdef _OPENMP
#include <omp.h>
int gact_oracle_num_threads(void) { return omp_get_max_threads(); }
void gact_oracle_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int gact_oracle_num_threads(void) { return 1; }
void gact_oracle_set_num_threads(int n) { (void)n; }
#endif
