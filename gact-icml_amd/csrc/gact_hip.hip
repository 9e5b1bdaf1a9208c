// GACT saved-activation compression for MI355X (gfx950): per-group min/max, scale, stochastic
// rounding, bit packing, and the inverse, as hand-written HIP kernels behind a C ABI.
//
// Quantize: a DPP row of 16 lanes owns one "super-group", the 8/bits consecutive groups of 256
// elements whose codes share output bytes.  Inside a group lane i of the row owns 16 columns in chunks
// of one 16-byte load each - float: 4 chunks of 4 columns at 4i + 64m, half: 2 chunks of 8 columns at
// 8i + 128m - so every load instruction of a row reads 256 contiguous bytes.  Per-group reductions are
// four row_ror DPP steps that never leave the row, and - because the reference packs the SAME column of
// 8/bits consecutive groups into one byte - the lane that owns a column owns every code of that byte:
// packing needs no cross-lane traffic at all.  One Philox block feeds 8 consecutive columns of two consecutive
// groups - a half chunk, or the float chunks of a pair of neighbouring lanes (which swap the words they need) -
// and, mirrored, the 8 columns half a group further on, which the same lane owns.
//
// Dequantize has no reduction, so a unit of 4 or 8 consecutive groups goes to a whole wave (float: lane l owns
// columns 4l .. 4l+3) or half a wave (half: 8l .. 8l+7): one 16-byte store per lane and group, every store
// instruction writing whole groups contiguously.  At 1, 2 and 4 bit the possible values of a unit (2^bits per
// group) are tabulated once across its lanes and fetched with ds_bpermute.  The stores are buffer stores whose
// cache policy the kernel chooses (nontemporal, written through at system scope).
//
// Element types: float and half as in the reference; bfloat16 (an addition) is quantized as the float
// values it holds, in the half layout.
//
// Workgroups are dealt to the 8 XCDs round-robin; xcd_tile() reorders the tiles so that each XCD's L2
// streams runs of consecutive tiles.
//
// Floating-point contract: this file is compiled with -ffp-contract=off, so every operation below is
// the IEEE operation it spells; the fused multiply-adds of the path are written __builtin_fmaf.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <queue>
#include <type_traits>
#include <utility>
#include <vector>

#include "gact_hip.h"

typedef _Float16 f16;
typedef __bf16 bf16;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define GROUP 256
#define ROW_GROUPS 8 /* groups of a dequantize unit and of a minimax row */

// ------------------------------------------------------------------------------------------------
// DPP row reductions (16 lanes).  Rotating by 8, 4, 2, 1 leaves the row-wide result in every lane.
// ------------------------------------------------------------------------------------------------
// Row-wide min of lo and max of hi, left in every lane of the row, with the rotated operand folded into the
// min / max instruction itself (VOP2 DPP).  lo and hi must not be NaN (they are per-lane results that
// started from a finite or infinite initial value).  A DPP operand has to be written two wait states before
// it is read, five after a vector write of EXEC; the compiler's hazard pass does not look inside an asm
// block, so the block keeps those distances itself, at both ends as well.
#define GACT_DPP_STEP(MIN, MAX, N)                                         \
  MIN " %0, %0, %0 row_ror:" #N " row_mask:0xf bank_mask:0xf\n\t"          \
  MAX " %1, %1, %1 row_ror:" #N " row_mask:0xf bank_mask:0xf\n\t"
#define GACT_DPP_ALL(MIN, MAX)                                             \
  "s_nop 4\n\t" GACT_DPP_STEP(MIN, MAX, 8) "s_nop 0\n\t" GACT_DPP_STEP(MIN, MAX, 4) "s_nop 0\n\t" \
  GACT_DPP_STEP(MIN, MAX, 2) "s_nop 0\n\t" GACT_DPP_STEP(MIN, MAX, 1) "s_nop 1"
__device__ __forceinline__ void row_all_minmax(float& lo, float& hi) {
  asm(GACT_DPP_ALL("v_min_f32_dpp", "v_max_f32_dpp") : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ void row_all_minmax(f16& lo, f16& hi) {
  asm(GACT_DPP_ALL("v_min_f16_dpp", "v_max_f16_dpp") : "+v"(lo), "+v"(hi));
}
// ------------------------------------------------------------------------------------------------
// Philox4x32.  The key schedule only depends on the seed, so it stays on the scalar unit; each
// round is two 32x32->64 multiplies and two three-input XORs (v_bitop3_b32, truth table 0x96).
// Ten rounds for the reference's stream (cuRAND's generator); seven for the fast stream - the fewest
// for which the generator's authors report that it passes BigCrush (Salmon et al., SC'11, table 2).
// ------------------------------------------------------------------------------------------------
#define PHILOX_REF_ROUNDS 10
#define PHILOX_FAST_ROUNDS 7
__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
}
template <int ROUNDS>
__device__ __forceinline__ void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                           uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int r = 0; r < ROUNDS; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = xor3((uint32_t)(p1 >> 32), c1, k0);
    uint32_t n2 = xor3((uint32_t)(p0 >> 32), c3, k1);
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// cuRAND's uniform map: float(x) * 2^-32 + 2^-33, in (0, 1].  The product is exact, so the fused form
// rounds once exactly like the separate multiply and add.
__device__ __forceinline__ float curand_uniform_map(uint32_t x) {
  return __builtin_fmaf((float)x, 0x1p-32f, 0x1p-33f);
}
// The same with the addend held in a register by the caller (uniform_addend(), once per kernel): left to itself the
// compiler builds the addend anew in front of every multiply-add, one instruction in nine of a kernel that is bound by
// its instruction count.
__device__ __forceinline__ float uniform_addend() {
  float c;
  asm volatile("v_mov_b32 %0, 0x2f000000" : "=v"(c));
  return c;
}
__device__ __forceinline__ float curand_uniform_map(uint32_t x, float addend) {
  float u;
  asm("v_fmamk_f32 %0, %1, 0x2f800000, %2" : "=v"(u) : "v"((float)x), "v"(addend));
  return u;
}
// 8-bit centred noise of the fast stream from byte B of a Philox word: (2h - 255) / 512 = (h + 0.5) / 256 - 1/2,
// exact in float (v_cvt_f32_ubyteB and one fma).
template <int B>
__device__ __forceinline__ float fast_centred_map(uint32_t w) {
  return __builtin_fmaf((float)((w >> (8 * B)) & 0xffu), 0x1p-8f, -255.0f / 512.0f);
}
__device__ __forceinline__ float fast_centred_map(uint32_t w, int b) {
  return (b & 2) ? ((b & 1) ? fast_centred_map<3>(w) : fast_centred_map<2>(w))
                 : ((b & 1) ? fast_centred_map<1>(w) : fast_centred_map<0>(w));
}

// Activations and codes are touched exactly once per kernel: load and store them with the streaming
// (nontemporal) hint so that they do not displace each other in L2 / Infinity Cache.
#ifndef GACT_STREAMING
#define GACT_STREAMING 1
#endif
template <typename V>
__device__ __forceinline__ V stream_load(const V* p) {
#if GACT_STREAMING
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}
template <typename V>
__device__ __forceinline__ void stream_store(V v, V* p) {
#if GACT_STREAMING
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

// The dequantized tensor leaves through buffer stores whose cache policy the kernel chooses: nontemporal, and for
// every type and width but float at 1 bit also written through at system scope (sc0 sc1 nt).  The plain nontemporal
// store the compiler emits for __builtin_nontemporal_store lets the L2 collect the lines first, which costs a float
// write stream up to 6 % (dequantize alone, buffers cold in every cache: 4 bit 103 M elements 75.5 -> 71.3 us, 256 M
// 183.4 -> 172.4; 8 bit 1 %; 2 bit equal; 17 M elements 1-3 % at every width; half 0-2 %), while float at 1 bit,
// whose stream has the smallest share of reads, loses 3-4 % by it from 50 M elements on (66.3 -> 68.5 us at 103 M)
// and keeps the plain nontemporal store on large tensors.
// A window is a buffer resource over the bytes from a wave-uniform base to the end of the tensor (at most 4 GB of
// them: offsets inside a window are 32 bit), so a store past the end of the tensor is dropped by the hardware.
#define GACT_STORE_NT 2          /* cache-policy bits of a buffer store: 1 sc0, 2 nt, 16 sc1 */
#define GACT_STORE_NT_SYSTEM 19
struct OutWindow {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ OutWindow(void* base, int64_t bytes) {
    const uint32_t n = bytes <= 0 ? 0u : bytes > 0xffffffffLL ? 0xffffffffu : (uint32_t)bytes;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)n, 0x00020000);
  }
  template <int POLICY>
  __device__ __forceinline__ void store16(u32x4 v, uint32_t byte_offset) const {
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (int)byte_offset, 0, POLICY);
  }
};
__device__ __forceinline__ int64_t wave_first(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// round-to-nearest-even integer of z clamped below at 0: rint(max(z, 0)) of the reference's
// __float2int_rn(fmax(z, 0)).  v_cvt_u32_f32 clamps negative inputs and NaN to 0, so no separate max is
// needed.  From 2^31 on the reference's signed conversion saturates to 0x7fffffff: SAT = true reproduces
// that (only min / max handed in by the caller can push a float code that far; with the group's own min
// and max a code stays below 2^bits + 1), SAT = false leaves it out.
template <bool SAT>
__device__ __forceinline__ uint32_t rint_clamp0(float z) {
  float r = __builtin_rintf(z);
  uint32_t c;
  asm("v_cvt_u32_f32_e32 %0, %1" : "=v"(c) : "v"(r));
  if (SAT) c = c < 0x7fffffffu ? c : 0x7fffffffu;
  return c;
}

// The same code read off the float.  For 0.5 <= y < 2^22, y - 0.5 is exact and adding 1.5 * 2^23 rounds it to
// 1.5 * 2^23 + rint(y - 0.5): in that binade a float's unit in the last place is 1, the constant is even, so
// ties go to even exactly as rint's do, and the integer sits in the low mantissa bits.  For 0 <= y < 0.5 the
// difference lies in [-0.5, 0) (possibly rounded, which cannot take it out of that interval) and the sum rounds
// to the constant itself: code 0, the reference's fmax.  NaN stays NaN with its payload: code 0 only where the
// payload's low byte is 0 - true of every NaN widened from half or bfloat16 and of the NaN arithmetic generates,
// not of any float NaN (the float path takes code_bits_of_any).
// Two additions; the bits above the code (0x4B4...) never reach the low 8 bits a byte keeps of a code shifted
// left by at most 7.  NOT valid for negative y (the callers' y is a sum of non-negative terms: with the group's own
// minimum no element lies below it) and for +inf, whose bits have a zero low byte where the reference's saturated
// conversion has 0xff: the one caller that can meet +inf (a half scale that overflowed) repairs those groups
// afterwards (quantize_supergroup).
__device__ __forceinline__ uint32_t code_bits_of(float y) {
  const float z = y - 0.5f;
  return __builtin_bit_cast(uint32_t, z + 12582912.0f);
}
// The same for any y: y + (2^23 - 0.5) rounds to 2^23 + rint(y - 0.5) in one step, and the median clamps to
// [2^23, 2^23 + 0x3fffff]: everything below 0.5, negative or NaN gives 0, +inf gives low bits of all ones.
__device__ __forceinline__ uint32_t clamp_code_bits(float w) {
  float c;
  asm("v_med3_f32 %0, %1, %2, %3" : "=v"(c) : "v"(w), "v"(8388608.0f), "v"(12582911.0f));
  return __builtin_bit_cast(uint32_t, c);
}
__device__ __forceinline__ uint32_t code_bits_of_any(float y) { return clamp_code_bits(y + 8388607.5f); }
// The fast stream adds a centred draw, so its sum z already is the reference's y - 0.5 and the code is rint(max(z, 0)):
// one addition (z > -0.5 with the group's own minimum, so z + 1.5 * 2^23 rounds to 1.5 * 2^23 + rint(z), -0 included),
// or the clamping form for any z.
__device__ __forceinline__ uint32_t centred_code_bits_of(float z) { return __builtin_bit_cast(uint32_t, z + 12582912.0f); }
__device__ __forceinline__ uint32_t centred_code_bits_of_any(float z) { return clamp_code_bits(z + 8388608.0f); }

// Correctly rounded c / s from the correctly rounded reciprocal r = RN(1/s) (Markstein): q = RN(c*r),
// e = c - s*q exactly (one FMA), result RN(q + e*r).  Valid for finite nonzero s with a normal quotient;
// the callers fall back to the division otherwise.
__device__ __forceinline__ float div_by_reciprocal(float c, float s, float r) {
  float q = c * r;
  float e = __builtin_fmaf(-q, s, c);
  return __builtin_fmaf(e, r, q);
}
// s is a scale the quotient c/s (0 <= c <= 255) can be taken through the reciprocal for: finite, and
// far enough from the ends of the exponent range that neither 1/s nor c/s is subnormal or overflows
__device__ __forceinline__ bool reciprocal_safe(float s) {
  float a = __builtin_fabsf(s);
  return a > 0x1p-100f && a < 0x1p100f;
}

// ------------------------------------------------------------------------------------------------
// Per-type pieces.  Store holds the 16 elements of one group a quantize lane owns (float: 4 chunks of 4,
// half and bfloat16: 2 chunks of 8).
// ------------------------------------------------------------------------------------------------
template <typename T> struct Elem;

template <> struct Elem<float> {
  // quantize layout: 4 chunks of 4 columns, 4i + 64m: one 16-byte load per chunk, 256 contiguous
  // bytes per row and load instruction
  static constexpr int kQChunks = 4, kQWidth = 4;
  static constexpr int kDtype = GACT_F32;
  typedef float Stat;   // type min, max and scale are computed and stored in (scale: always; min: as T)
  __device__ static __forceinline__ float stat_of(float x) { return x; }
  __device__ static __forceinline__ float elem_of(float x) { return x; }
  struct Store { float v[4][4]; };
  __device__ static __forceinline__ void load_noise(const float* p, float (&u)[4]) {
    f32x4 a = stream_load(reinterpret_cast<const f32x4*>(p));
    u[0] = a.x; u[1] = a.y; u[2] = a.z; u[3] = a.w;
  }
  __device__ static __forceinline__ void load_chunk(const float* p, Store& st, int k) { load_noise(p, st.v[k]); }
  __device__ static __forceinline__ void set(Store& st, int k, int e, float x) { st.v[k][e] = x; }
  __device__ static __forceinline__ float init_lo() { return 1e30f; }
  __device__ static __forceinline__ float init_hi() { return -1e30f; }
  __device__ static __forceinline__ float from_float(float v) { return v; }
  // min and max of the whole group, in every lane of the row
  __device__ static __forceinline__ void group_minmax(const Store& st, float& lo_out, float& hi_out) {
    float lo = init_lo(), hi = init_hi();
#pragma unroll
    for (int k = 0; k < kQChunks; k++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        lo = __builtin_fminf(lo, st.v[k][e]);
        hi = __builtin_fmaxf(hi, st.v[k][e]);
      }
    row_all_minmax(lo, hi);
    lo_out = lo;
    hi_out = hi;
  }
  __device__ static __forceinline__ void store_codes(uint8_t* p, const uint32_t (&b)[4]) {
    // the reference accumulates in a uint8_t: keep the low 8 bits of every byte
    uint32_t w = (b[0] & 0xffu) | ((b[1] & 0xffu) << 8) | ((b[2] & 0xffu) << 16) | (b[3] << 24);
    stream_store(w, reinterpret_cast<uint32_t*>(p));
  }
  // scale = float( double(float(qmax)) / (double(max - min) + 2e-6) )
  __device__ static __forceinline__ float make_scale(float lo, float hi, int qmax) {
    float range = hi - lo;
    return (float)((double)(float)qmax / ((double)range + 2e-6));
  }
  // code = rint(max(fma(x - mn, s, u) - 0.5, 0)).  ANY = true: min and scale may be anything (the pack entry
  // point), the code is converted as the reference converts it; ANY = false: they are the group's own, the
  // sum stays below 2^bits + 1 and the code is read off the float (code_bits_of: its low 8 bits count)
  // CENTRED: u is a centred draw of the fast stream (the - 0.5 is in it)
  template <bool ANY, bool CENTRED = false>
  __device__ static __forceinline__ uint32_t code1(const Store& st, int k, int e, float mn, float s, float u) {
    float t = st.v[k][e] - mn;
    float y = __builtin_fmaf(t, s, u);
    // a NaN element keeps its payload through the subtraction and the fma, and a payload may have anything in its
    // low byte: the clamping form (code 0 for every NaN, like the reference's fmax) rather than code_bits_of
    if (CENTRED) return ANY ? rint_clamp0<true>(y) : centred_code_bits_of_any(y);
    return ANY ? rint_clamp0<true>(y - 0.5f) : code_bits_of_any(y);
  }
  // elements e (even) and e + 1 of chunk k
  template <bool ANY>
  __device__ static __forceinline__ void code2(const Store& st, int k, int e, float mn, float s, float ua, float ub,
                                               uint32_t& ca, uint32_t& cb) {
    ca = code1<ANY>(st, k, e, mn, s, ua);
    cb = code1<ANY>(st, k, e + 1, mn, s, ub);
  }
  // NEG (with CENTRED): the chunk takes the mirrored draws, -u (the negation folds into the fma)
  template <bool CONST_NOISE, bool ANY, bool CENTRED = false, bool NEG = false>
  __device__ static __forceinline__ void codes(const Store& st, int k, float mn, float s, const float (&u)[4],
                                               uint32_t (&c)[4]) {
#pragma unroll
    for (int e = 0; e < 4; e++) c[e] = code1<ANY, CENTRED>(st, k, e, mn, s, NEG ? -u[e] : u[e]);
  }
  // a float scale is never infinite (the denominator is at least 2e-6) and with the group's own min and max the
  // sum stays finite: nothing to repair
  static constexpr bool kRepairsInfiniteScale = false;
  __device__ static __forceinline__ bool scale_is_inf(float) { return false; }
  __device__ static __forceinline__ bool above(const Store&, int, int, float) { return false; }

  // ---- dequantize: out = float(code) / scale + min ----
  struct Dq { float s, r, mn; bool fast; };
  __device__ static __forceinline__ Dq dq_prepare(float s, float mn) {
    Dq d;
    d.s = s; d.mn = mn;
    d.fast = reciprocal_safe(s);
    d.r = 1.0f / s;
    return d;
  }
  __device__ static __forceinline__ float decode(int c, const Dq& d) {
    float q = d.fast ? div_by_reciprocal((float)c, d.s, d.r) : (float)c / d.s;
    return q + d.mn;
  }
  // quotient -> output; one table entry T(c)/scale + min; 32 bits fetched from another lane -> value
  __device__ static __forceinline__ float finish(float q, float mn) { return q + mn; }
  __device__ static __forceinline__ uint32_t table_entry(float c, float s, float mn) {
    return __builtin_bit_cast(uint32_t, c / s + mn);
  }
  __device__ static __forceinline__ float from_bits(uint32_t b) { return __builtin_bit_cast(float, b); }
  static constexpr int kDqWidth = 4;  // columns per dequantize lane: one 16-byte store
  template <int POLICY>
  __device__ static __forceinline__ void store_dq(const OutWindow& w, uint32_t byte_offset, const float (&v)[4]) {
    f32x4 a = {v[0], v[1], v[2], v[3]};
    w.template store16<POLICY>(__builtin_bit_cast(u32x4, a), byte_offset);
  }
};

template <> struct Elem<f16> {
  // quantize layout: 2 chunks of 8 columns, 8i + 128m: one 16-byte load per chunk
  static constexpr int kQChunks = 2, kQWidth = 8;
  static constexpr int kDtype = GACT_F16;
  typedef f16 Stat;
  __device__ static __forceinline__ f16 stat_of(f16 x) { return x; }
  __device__ static __forceinline__ f16 elem_of(f16 x) { return x; }
  struct Store { f16x2 v[2][4]; };   // pairs, so that subtraction and product run as packed ops
  __device__ static __forceinline__ void store_codes(uint8_t* p, const uint32_t (&b)[8]) {
    u32x2 w;
    w.x = (b[0] & 0xffu) | ((b[1] & 0xffu) << 8) | ((b[2] & 0xffu) << 16) | (b[3] << 24);
    w.y = (b[4] & 0xffu) | ((b[5] & 0xffu) << 8) | ((b[6] & 0xffu) << 16) | (b[7] << 24);
    stream_store(w, reinterpret_cast<u32x2*>(p));
  }
  __device__ static __forceinline__ void load_noise(const float* p, float (&u)[8]) {
    f32x4 a = stream_load(reinterpret_cast<const f32x4*>(p));
    f32x4 b = stream_load(reinterpret_cast<const f32x4*>(p + 4));
    u[0] = a.x; u[1] = a.y; u[2] = a.z; u[3] = a.w;
    u[4] = b.x; u[5] = b.y; u[6] = b.z; u[7] = b.w;
  }
  __device__ static __forceinline__ void load_chunk(const f16* p, Store& st, int k) {
    f16x8 a = stream_load(reinterpret_cast<const f16x8*>(p));
#pragma unroll
    for (int j = 0; j < 4; j++) st.v[k][j] = f16x2{a[2 * j], a[2 * j + 1]};
  }
  __device__ static __forceinline__ void set(Store& st, int k, int e, f16 x) { st.v[k][e >> 1][e & 1] = x; }
  __device__ static __forceinline__ float init_lo() { return __builtin_inff(); }  // half(1e30) is +inf
  __device__ static __forceinline__ float init_hi() { return -__builtin_inff(); }
  __device__ static __forceinline__ f16 from_float(float v) { return (f16)v; }
  // Packed min / max without the canonicalising copy the compiler puts in front of every minnum / maxnum
  // operand: a quiet NaN operand loses against the other one, which is the reference's "NaN is ignored".
  // (A signalling NaN, which arithmetic never produces, would be returned quieted instead.)
  __device__ static __forceinline__ f16x2 pk_min(f16x2 a, f16x2 b) {
    f16x2 d;
    asm("v_pk_min_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
  }
  __device__ static __forceinline__ f16x2 pk_max(f16x2 a, f16x2 b) {
    f16x2 d;
    asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
  }
  // min and max of the whole group, in every lane of the row: packed per-lane min / max from +-inf (the
  // start values only survive in a lane whose 16 elements are all NaN), the two halves against each other,
  // then the row reduction
  __device__ static __forceinline__ void group_minmax(const Store& st, f16& lo_out, f16& hi_out) {
    const f16 inf = (f16)__builtin_inff();
    f16x2 l = {inf, inf}, h = {(f16)-inf, (f16)-inf};
#pragma unroll
    for (int k = 0; k < kQChunks; k++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        l = pk_min(l, st.v[k][j]);
        h = pk_max(h, st.v[k][j]);
      }
    f16 lo, hi;
    asm("v_min_f16_sdwa %0, %1, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1"
        : "=v"(lo) : "v"(l));
    asm("v_max_f16_sdwa %0, %1, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1"
        : "=v"(hi) : "v"(h));
    row_all_minmax(lo, hi);
    lo_out = lo;
    hi_out = hi;
  }
  // range is a half operation; the quotient is a double narrowed to float and then to half
  __device__ static __forceinline__ f16 make_scale(f16 lo, f16 hi, int qmax) {
    f16 range = hi - lo;
    return (f16)(float)((double)(float)qmax / ((double)(float)range + 2e-6));
  }
  // float(p) + u with p taken from the low / high half of a pair: one v_fma_mix_f32 (p * 1.0 + u)
  __device__ static __forceinline__ float widen_add_lo(f16x2 p, float u) {
    float y;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(y) : "v"(p), "v"(u));
    return y;
  }
  __device__ static __forceinline__ float widen_add_hi(f16x2 p, float u) {
    float y;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(y) : "v"(p), "v"(u));
    return y;
  }
  // float(p) - u: the same instruction with the addend's sign flipped
  __device__ static __forceinline__ float widen_sub_lo(f16x2 p, float u) {
    float y;
    asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(y) : "v"(p), "v"(u));
    return y;
  }
  __device__ static __forceinline__ float widen_sub_hi(f16x2 p, float u) {
    float y;
    asm("v_fma_mix_f32 %0, %1, 1.0, -%2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(y) : "v"(p), "v"(u));
    return y;
  }
  // half subtraction and half product (each rounded to half), then float: y = float(p) + u,
  // code = rint(max(y - 0.5, 0)).  |y| <= 65505 or y is infinite or NaN whatever min and scale are, so the
  // code is always read off the float.  ANY = true (min and scale from the caller): y may be negative or +inf,
  // the clamping form takes both.  ANY = false: y >= 0, and where it is +inf (the scale overflowed to inf)
  // the caller repairs the group afterwards.
  template <bool ANY, bool CENTRED = false>
  __device__ static __forceinline__ uint32_t code1(const Store& st, int k, int e, f16 mn, f16 s, float u) {
    f16 t = st.v[k][e >> 1][e & 1] - mn;
    f16 p = t * s;
    float y = (float)p + u;
    if (CENTRED) return ANY ? centred_code_bits_of_any(y) : centred_code_bits_of(y);
    return ANY ? code_bits_of_any(y) : code_bits_of(y);
  }
  // elements e (even) and e + 1 of chunk k, one pair: packed subtraction and product, the sum with the widening folded in
  template <bool ANY>
  __device__ static __forceinline__ void code2(const Store& st, int k, int e, f16 mn, f16 s, float ua, float ub,
                                               uint32_t& ca, uint32_t& cb) {
    const f16x2 mn2 = {mn, mn}, s2 = {s, s};
    const f16x2 p = (st.v[k][e >> 1] - mn2) * s2;
    const float ya = widen_add_lo(p, ua), yb = widen_add_hi(p, ub);
    ca = ANY ? code_bits_of_any(ya) : code_bits_of(ya);
    cb = ANY ? code_bits_of_any(yb) : code_bits_of(yb);
  }
  template <bool CONST_NOISE, bool ANY, bool CENTRED = false, bool NEG = false>
  __device__ static __forceinline__ void codes(const Store& st, int k, f16 mn, f16 s, const float (&u)[8],
                                               uint32_t (&c)[8]) {
    const f16x2 mn2 = {mn, mn}, s2 = {s, s};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      f16x2 t = st.v[k][j] - mn2;
      f16x2 p = t * s2;
      if (CENTRED) {
        // the fast stream: float(p) +- c in one v_fma_mix_f32, then the code off the float
        const float zl = NEG ? widen_sub_lo(p, u[2 * j]) : widen_add_lo(p, u[2 * j]);
        const float zh = NEG ? widen_sub_hi(p, u[2 * j + 1]) : widen_add_hi(p, u[2 * j + 1]);
        c[2 * j] = ANY ? centred_code_bits_of_any(zl) : centred_code_bits_of(zl);
        c[2 * j + 1] = ANY ? centred_code_bits_of_any(zh) : centred_code_bits_of(zh);
      } else if (CONST_NOISE) {
        // u = 0.5: float(p) + 0.5 and the following - 0.5 are both exact for every half p (at most 24
        // significant bits between 2^-1 and p's last bit), so y - 0.5 == float(p) and the code is
        // rint(float(p)): float(p) plus the constant rounds to the constant + rint(float(p))
        if (ANY) {
          c[2 * j] = clamp_code_bits(widen_add_lo(p, 8388608.0f));
          c[2 * j + 1] = clamp_code_bits(widen_add_hi(p, 8388608.0f));
        } else {
          c[2 * j] = __builtin_bit_cast(uint32_t, widen_add_lo(p, 12582912.0f));
          c[2 * j + 1] = __builtin_bit_cast(uint32_t, widen_add_hi(p, 12582912.0f));
        }
      } else if (ANY) {
        c[2 * j] = code_bits_of_any(widen_add_lo(p, u[2 * j]));
        c[2 * j + 1] = code_bits_of_any(widen_add_hi(p, u[2 * j + 1]));
      } else {
        c[2 * j] = code_bits_of(widen_add_lo(p, u[2 * j]));
        c[2 * j + 1] = code_bits_of(widen_add_hi(p, u[2 * j + 1]));
      }
    }
  }
  // Where the scale is +inf every element above the minimum has an infinite product, whose code the reference
  // saturates to 0x7fffffff: all ones from the element's field upwards.  (An element equal to the minimum gives
  // 0 * inf = NaN: code 0.)  code_bits_of leaves 0 in both cases; this adds the ones.
  static constexpr bool kRepairsInfiniteScale = true;
  __device__ static __forceinline__ bool scale_is_inf(f16 s) { return __builtin_isinf((float)s); }
  __device__ static __forceinline__ bool above(const Store& st, int k, int e, f16 mn) { return st.v[k][e >> 1][e & 1] > mn; }

  // ---- dequantize: half(code) / scale is a float division rounded to half; the sum is rounded to half ----
  struct Dq { float s, r; f16 mn; bool fast; };
  __device__ static __forceinline__ Dq dq_prepare(f16 s, f16 mn) {
    Dq d;
    d.s = (float)s; d.mn = mn;
    d.fast = reciprocal_safe(d.s);
    d.r = 1.0f / d.s;
    return d;
  }
  __device__ static __forceinline__ f16 decode(int c, const Dq& d) {
    float q = d.fast ? div_by_reciprocal((float)c, d.s, d.r) : (float)c / d.s;
    return (f16)q + d.mn;
  }
  __device__ static __forceinline__ f16 finish(float q, f16 mn) { return (f16)q + mn; }
  __device__ static __forceinline__ uint32_t table_entry(float c, f16 s, f16 mn) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (f16)((f16)(c / (float)s) + mn));
  }
  __device__ static __forceinline__ f16 from_bits(uint32_t b) { return __builtin_bit_cast(f16, (uint16_t)b); }
  static constexpr int kDqWidth = 8;  // columns per dequantize lane: one 16-byte store
  template <int POLICY>
  __device__ static __forceinline__ void store_dq(const OutWindow& w, uint32_t byte_offset, const f16 (&v)[8]) {
    f16x8 a;
#pragma unroll
    for (int e = 0; e < 8; e++) a[e] = v[e];
    w.template store16<POLICY>(__builtin_bit_cast(u32x4, a), byte_offset);
  }
};

// bfloat16 (not in the reference, which knows float and half): every bfloat16 is a float, so the group is
// widened on load and quantized exactly as the float path quantizes those floats - same min, same float
// scale, same codes - with the half layout (8-column chunks, one 16-byte load each).  The scale is kept in
// float (8 significant bits would not do), the minimum is one of the inputs and goes back to bfloat16
// unchanged, and dequantize rounds float(code) / scale + min to bfloat16 once, to nearest even.
template <> struct Elem<bf16> {
  static constexpr int kQChunks = 2, kQWidth = 8;
  static constexpr int kDtype = GACT_BF16;
  typedef float Stat;
  __device__ static __forceinline__ float stat_of(bf16 x) { return (float)x; }
  __device__ static __forceinline__ bf16 elem_of(float x) { return (bf16)x; }
  // the group stays in registers as loaded (pairs of bfloat16) and is widened where it is used - once for
  // min / max, once for the codes: half the registers of a widened copy (1 bit: 8 groups per lane)
  struct Store { uint32_t w[2][4]; };
  __device__ static __forceinline__ float widen(const Store& st, int k, int e) {
    const uint32_t w = st.w[k][e >> 1];
    return __builtin_bit_cast(float, (e & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  __device__ static __forceinline__ void store_codes(uint8_t* p, const uint32_t (&b)[8]) { Elem<f16>::store_codes(p, b); }
  __device__ static __forceinline__ void load_noise(const float* p, float (&u)[8]) { Elem<f16>::load_noise(p, u); }
  __device__ static __forceinline__ void load_chunk(const bf16* p, Store& st, int k) {
    const u32x4 a = stream_load(reinterpret_cast<const u32x4*>(p));
    st.w[k][0] = a.x; st.w[k][1] = a.y; st.w[k][2] = a.z; st.w[k][3] = a.w;
  }
  __device__ static __forceinline__ void set(Store& st, int k, int e, bf16 x) {
    const uint32_t h = (uint32_t)__builtin_bit_cast(uint16_t, x);
    if (e & 1) st.w[k][e >> 1] |= h << 16;   // the callers set a chunk's elements in order: the even one starts the pair
    else st.w[k][e >> 1] = h;
  }
  __device__ static __forceinline__ void group_minmax(const Store& st, float& lo_out, float& hi_out) {
    float lo = Elem<float>::init_lo(), hi = Elem<float>::init_hi();
#pragma unroll
    for (int k = 0; k < kQChunks; k++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        lo = __builtin_fminf(lo, widen(st, k, e));
        hi = __builtin_fmaxf(hi, widen(st, k, e));
      }
    row_all_minmax(lo, hi);
    lo_out = lo;
    hi_out = hi;
  }
  __device__ static __forceinline__ float make_scale(float lo, float hi, int qmax) {
    return Elem<float>::make_scale(lo, hi, qmax);
  }
  template <bool ANY, bool CENTRED = false>
  __device__ static __forceinline__ uint32_t code1(const Store& st, int k, int e, float mn, float s, float u) {
    float t = widen(st, k, e) - mn;
    float y = __builtin_fmaf(t, s, u);
    if (CENTRED) return ANY ? rint_clamp0<true>(y) : centred_code_bits_of(y);
    return ANY ? rint_clamp0<true>(y - 0.5f) : code_bits_of(y);
  }
  template <bool ANY>
  __device__ static __forceinline__ void code2(const Store& st, int k, int e, float mn, float s, float ua, float ub,
                                               uint32_t& ca, uint32_t& cb) {
    ca = code1<ANY>(st, k, e, mn, s, ua);
    cb = code1<ANY>(st, k, e + 1, mn, s, ub);
  }
  template <bool CONST_NOISE, bool ANY, bool CENTRED = false, bool NEG = false>
  __device__ static __forceinline__ void codes(const Store& st, int k, float mn, float s, const float (&u)[8],
                                               uint32_t (&c)[8]) {
#pragma unroll
    for (int e = 0; e < 8; e++) c[e] = code1<ANY, CENTRED>(st, k, e, mn, s, NEG ? -u[e] : u[e]);
  }
  static constexpr bool kRepairsInfiniteScale = false;
  __device__ static __forceinline__ bool scale_is_inf(float) { return false; }
  __device__ static __forceinline__ bool above(const Store&, int, int, float) { return false; }
  __device__ static __forceinline__ bf16 finish(float q, float mn) { return (bf16)(q + mn); }
  __device__ static __forceinline__ uint32_t table_entry(float c, float s, float mn) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (bf16)(c / s + mn));
  }
  __device__ static __forceinline__ bf16 from_bits(uint32_t b) { return __builtin_bit_cast(bf16, (uint16_t)b); }
  static constexpr int kDqWidth = 8;
  template <int POLICY>
  __device__ static __forceinline__ void store_dq(const OutWindow& w, uint32_t byte_offset, const bf16 (&v)[8]) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    bf16x8 a;
#pragma unroll
    for (int e = 0; e < 8; e++) a[e] = v[e];
    w.template store16<POLICY>(__builtin_bit_cast(u32x4, a), byte_offset);
  }
};

// Column of the first element of chunk k for row lane i: chunks are W columns wide and 16*W apart.
template <typename T>
__device__ __forceinline__ int chunk_col(int k, int i) { return Elem<T>::kQWidth * (16 * k + i); }

// Load the 16 elements lane i owns of group n; elements at or beyond numel read as zero (the zero
// padding of gact/gact/ops.py:12-17 without the copy).
template <typename T>
__device__ __forceinline__ void load_group(const T* __restrict__ x, int64_t numel, int64_t n, int i,
                                           typename Elem<T>::Store& st) {
  constexpr int CH = Elem<T>::kQChunks, W = Elem<T>::kQWidth;
  const int64_t base = n * GROUP;
  if (base + GROUP <= numel) {
#pragma unroll
    for (int k = 0; k < CH; k++) Elem<T>::load_chunk(x + base + chunk_col<T>(k, i), st, k);
  } else {
#pragma unroll
    for (int k = 0; k < CH; k++)
#pragma unroll
      for (int e = 0; e < W; e++) {
        int64_t idx = base + chunk_col<T>(k, i) + e;
        Elem<T>::set(st, k, e, idx < numel ? x[idx] : (T)0.0f);
      }
  }
}

// value of lane LANE of the row, in every lane of the row (DPP row_newbcast)
template <int LANE>
__device__ __forceinline__ uint32_t row_bcast_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x150 + LANE, 0xf, 0xf, false);
}
template <int LANE> __device__ __forceinline__ float row_bcast(float v) {
  return __builtin_bit_cast(float, row_bcast_u32<LANE>(__builtin_bit_cast(uint32_t, v)));
}
template <int LANE> __device__ __forceinline__ f16 row_bcast(f16 v) {
  return __builtin_bit_cast(f16, (uint16_t)row_bcast_u32<LANE>((uint32_t)__builtin_bit_cast(uint16_t, v)));
}

// swap with the neighbouring lane (lane ^ 1): DPP quad_perm [1,0,3,2]
__device__ __forceinline__ uint32_t swap_with_neighbour(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0xB1, 0xf, 0xf, false);
}

// The fast stream.  Two consecutive groups (512 elements) draw 16 Philox blocks; block j serves columns 8j .. 8j+7 of
// both: its bytes 0..7 (word by word, low byte first) the first group's, bytes 8..15 the second's, one byte h per
// element, taken as the centred draw c = (2h - 255) / 512.  The column 128 further on takes -c, the same draw
// mirrored: every element's noise is uniform on the same 256-point grid, symmetric about 0 and strictly inside
// (-1/2, 1/2), and the two elements of a pair (which sit half a group apart) round in opposite directions more
// often than not (their rounding errors have covariance <= 0).  One block per 32 elements, one conversion and one
// fma per two elements (the mirrored draw is a sign flip that folds into the instruction that adds it).
// In terms of the flat element index E: block (E / 512) * 16 + (E % 128) / 8, byte ((E / 256) % 2) * 8 + E % 8,
// mirrored if E % 256 >= 128.
__device__ __forceinline__ uint64_t fast_block_of(uint64_t E) { return (E >> 9) * 16 + ((E & 127) >> 3); }
// the centred draw of element E from the words of its block
__device__ __forceinline__ float fast_centred_of(const uint32_t (&r)[4], uint64_t E) {
  const int b = (int)(((E >> 8) & 1) * 8 + (E & 7));
  const uint32_t w = (b & 8) ? ((b & 4) ? r[3] : r[2]) : ((b & 4) ? r[1] : r[0]);
  const float c = fast_centred_map(w, b & 3);
  return (E & 128) ? -c : c;
}

// The two words of each group of the pair `pair` that row lane i needs: w[g][0..1] hold the 8 draws of the lane's
// unmirrored columns of group 2 * pair + g, in column order.  With 8-column chunks (8i + 128m) that is the lane's
// own block.  With 4-column chunks (4i + 64m) chunks 0 and 1 are halves of blocks i/2 and 8 + i/2, which two
// neighbouring lanes share: the even lane computes the first, the odd lane the second, and they exchange the words
// the other one needs (the even lane owns words 0 and 2 of a block, the odd lane words 1 and 3).
template <typename T>
__device__ __forceinline__ void fast_pair_words(int64_t pair, int i, uint32_t k0, uint32_t k1, uint32_t (&w)[2][2]) {
  constexpr int CH = Elem<T>::kQChunks, W = Elem<T>::kQWidth;
  uint32_t r[4];
  if (W == 8) {
    static_assert(W != 8 || CH == 2, "two chunks of 8 columns, 128 apart");
    const uint64_t blk = (uint64_t)pair * 16 + i;
    philox4x32<PHILOX_FAST_ROUNDS>(0u, 0u, (uint32_t)blk, (uint32_t)(blk >> 32), k0, k1, r);
    w[0][0] = r[0]; w[0][1] = r[1]; w[1][0] = r[2]; w[1][1] = r[3];
  } else {
    static_assert(W == 8 || CH == 4, "four chunks of 4 columns, 64 apart");
    const bool odd = i & 1;
    const uint64_t blk = (uint64_t)pair * 16 + (odd ? 8 : 0) + (i >> 1);
    philox4x32<PHILOX_FAST_ROUNDS>(0u, 0u, (uint32_t)blk, (uint32_t)(blk >> 32), k0, k1, r);
    const uint32_t g0 = swap_with_neighbour(odd ? r[0] : r[1]);
    const uint32_t g1 = swap_with_neighbour(odd ? r[2] : r[3]);
    w[0][0] = odd ? g0 : r[0];   // chunk 0: block i/2
    w[0][1] = odd ? r[1] : g0;   // chunk 1: block 8 + i/2
    w[1][0] = odd ? g1 : r[2];
    w[1][1] = odd ? r[3] : g1;
  }
}
// The centred draws of the lane's unmirrored chunks (the first half of its chunks) from the group's two words: draw
// k * W + e belongs to element e of chunk k; chunk k + CH/2 takes the same draws negated.
template <typename T>
__device__ __forceinline__ void fast_centred_draws(const uint32_t (&w)[2], float (&c)[Elem<T>::kQChunks / 2][Elem<T>::kQWidth]) {
  constexpr int CH = Elem<T>::kQChunks, W = Elem<T>::kQWidth;
#pragma unroll
  for (int k = 0; k < CH / 2; k++)
#pragma unroll
    for (int e = 0; e < W; e++) {
      const int f = k * W + e;
      c[k][e] = (f & 2) ? ((f & 1) ? fast_centred_map<3>(w[f >> 2]) : fast_centred_map<2>(w[f >> 2]))
                        : ((f & 1) ? fast_centred_map<1>(w[f >> 2]) : fast_centred_map<0>(w[f >> 2]));
    }
}
// The state of the fast stream along a row's groups: group g of the row (first group n0) draws from the words of its
// pair, which are computed when the row enters the pair.  Rows of two or more groups start on an even group, so that
// happens at every even g; a row of one group computes its pair's block and takes its half.
template <typename T, int GPR>
struct FastRow {
  uint32_t w[2][2];
  __device__ __forceinline__ void draws(int g, int64_t n0, int i, uint32_t k0, uint32_t k1,
                                        float (&c)[Elem<T>::kQChunks / 2][Elem<T>::kQWidth]) {
    if (GPR == 1) {
      const int64_t n = n0 + g;
      fast_pair_words<T>(n >> 1, i, k0, k1, w);
      const uint32_t mine[2] = {(n & 1) ? w[1][0] : w[0][0], (n & 1) ? w[1][1] : w[0][1]};
      fast_centred_draws<T>(mine, c);
    } else {
      if ((g & 1) == 0) fast_pair_words<T>((n0 + g) >> 1, i, k0, k1, w);
      fast_centred_draws<T>(w[g & 1], c);
    }
  }
};

// ------------------------------------------------------------------------------------------------
// Quantize SGR consecutive super-groups (one 16-lane row): all their groups are loaded first, reduced, and share
// one scale division per lane; the codes then go out super-group by super-group.
//   STAGE > 0 (rows of whole groups): STAGE groups at a time instead, see below; LAZY: each stage issues its own loads.
//   GIVEN = false: min/max are reduced here (fused minimax + scale + pack, one read of x).
//   GIVEN = true : min/max are read from mn_io / mx_io (the pack entry point's contract).
// Codes follow quantization_cuda_kernel.cu:38-71; see Elem<T>::code1 for the arithmetic.
// ------------------------------------------------------------------------------------------------
template <typename T, int BITS, int NOISE, bool GIVEN, int SGR = 1, int STAGE = 0, bool LAZY = false>
__device__ __forceinline__ void quantize_supergroup(const T* __restrict__ x, int64_t numel, int64_t N, int64_t sg0,
                                                    int i, uint8_t* __restrict__ packed,
                                                    typename Elem<T>::Stat* __restrict__ scale_out,
                                                    T* mn_io, T* mx_io, uint32_t k0, uint32_t k1,
                                                    const float* __restrict__ noise) {
  constexpr int WPT = 8 / BITS;
  constexpr int GPR = SGR * WPT;   // groups of the row
  static_assert(GPR == 1 || GPR == 2 || GPR == 4 || GPR == 8, "a row holds 1, 2, 4 or 8 groups");
  constexpr int QMAX = (1 << BITS) - 1;
  constexpr int CH = Elem<T>::kQChunks, W = Elem<T>::kQWidth;
  const int64_t n0 = sg0 * WPT;

  typename Elem<T>::Store v[GPR];
  typedef typename Elem<T>::Stat Stat;
  Stat lo_t[GPR], hi_t[GPR], s_t[GPR];
  // The staged path is for rows of whole groups.  The choice is made for the wave, not for the row: a wave in which
  // one row is ragged (the tensor's last) would otherwise run both paths one after the other, each with its own
  // round trip to memory - and being the tensor's last wave it would hold up the end of the kernel.
  const bool whole_row = (n0 + GPR) * GROUP <= numel;
  if (STAGE > 0 && STAGE < GPR && !GIVEN && NOISE != GACT_NOISE_REF && __builtin_amdgcn_ballot_w64(!whole_row) == 0) {
    // All groups whole: the loads in one straight line, then STAGE groups at a time as they arrive: reduce, divide
    // (lane j for group j % STAGE of the stage), encode; a super-group goes out when its last group is done.  The
    // work on the first groups overlaps the loads of the later ones within the wave, which pays where few waves
    // share a SIMD (small tensors) and costs the extra divisions elsewhere.  LAZY: a stage's loads are issued when
    // the stage begins (the compiler still hoists what its register budget allows), which suits the
    // instruction-heavy half kernels once several waves share a SIMD.
    static_assert(STAGE <= 0 || (GPR % (STAGE > 0 ? STAGE : 1) == 0 && (STAGE & (STAGE - 1)) == 0), "stages divide the row");
    constexpr int ST = STAGE > 0 ? STAGE : 1;
    if (!LAZY) {
#pragma unroll
      for (int g = 0; g < GPR; g++)
#pragma unroll
        for (int k = 0; k < CH; k++) Elem<T>::load_chunk(x + (n0 + g) * GROUP + chunk_col<T>(k, i), v[g], k);
    }
    uint32_t bytes[CH][W];
    FastRow<T, GPR> fast;
#pragma unroll
    for (int g0 = 0; g0 < GPR; g0 += ST) {
      if (LAZY) {
#pragma unroll
        for (int j = 0; j < ST; j++)
#pragma unroll
          for (int k = 0; k < CH; k++) Elem<T>::load_chunk(x + (n0 + g0 + j) * GROUP + chunk_col<T>(k, i), v[g0 + j], k);
      }
      Stat lo_s[ST], hi_s[ST], sc_s[ST];
#pragma unroll
      for (int j = 0; j < ST; j++) {
        lo_s[j] = hi_s[j] = (Stat)0.0f;
        Elem<T>::group_minmax(v[g0 + j], lo_s[j], hi_s[j]);
      }
      {
        const int mine = i & (ST - 1);
        Stat lo_m = lo_s[0], hi_m = hi_s[0];
#pragma unroll
        for (int j = 1; j < ST; j++) {
          lo_m = (mine == j) ? lo_s[j] : lo_m;
          hi_m = (mine == j) ? hi_s[j] : hi_m;
        }
        const Stat s_m = Elem<T>::make_scale(lo_m, hi_m, QMAX);
        if (i < ST) {
          scale_out[n0 + g0 + i] = s_m;
          mn_io[n0 + g0 + i] = Elem<T>::elem_of(lo_m);
          if (mx_io) mx_io[n0 + g0 + i] = Elem<T>::elem_of(hi_m);
        }
        if (ST == 1) {
          sc_s[0] = s_m;
        } else {
          sc_s[0] = row_bcast<0>(s_m);
          sc_s[1 % ST] = row_bcast<1>(s_m);
          if (ST > 2) { sc_s[2 % ST] = row_bcast<2>(s_m); sc_s[3 % ST] = row_bcast<3>(s_m); }
        }
      }
#pragma unroll
      for (int j = 0; j < ST; j++) {
        const int g = g0 + j;
        const int64_t n = n0 + g;
        const int ni = g % WPT;
        if (ni == 0) {
#pragma unroll
          for (int k = 0; k < CH; k++)
#pragma unroll
            for (int e = 0; e < W; e++) bytes[k][e] = 0;
        }
        if (NOISE == GACT_NOISE_FAST) {
          float cd[CH / 2][W];
          fast.draws(g, n0, i, k0, k1, cd);
#pragma unroll
          for (int k = 0; k < CH; k++) {
            uint32_t c[W];
            if (k < CH / 2) Elem<T>::template codes<false, GIVEN, true, false>(v[g], k, lo_s[j], sc_s[j], cd[k % (CH / 2)], c);
            else Elem<T>::template codes<false, GIVEN, true, true>(v[g], k, lo_s[j], sc_s[j], cd[k % (CH / 2)], c);
#pragma unroll
            for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << (ni * BITS);
          }
        } else {
          float u[CH][W];
#pragma unroll
          for (int k = 0; k < CH; k++) {
            if (NOISE == GACT_NOISE_INJECT) {
              Elem<T>::load_noise(noise + n * GROUP + chunk_col<T>(k, i), u[k]);
            } else {
#pragma unroll
              for (int e = 0; e < W; e++) u[k][e] = 0.5f;
            }
          }
#pragma unroll
          for (int k = 0; k < CH; k++) {
            uint32_t c[W];
            Elem<T>::template codes<NOISE == GACT_NOISE_CONST, GIVEN>(v[g], k, lo_s[j], sc_s[j], u[k], c);
#pragma unroll
            for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << (ni * BITS);
          }
        }
        if (Elem<T>::kRepairsInfiniteScale && __builtin_amdgcn_ballot_w64(Elem<T>::scale_is_inf(sc_s[j])) != 0) {
          if (Elem<T>::scale_is_inf(sc_s[j])) {
#pragma unroll
            for (int k = 0; k < CH; k++)
#pragma unroll
              for (int e = 0; e < W; e++)
                if (Elem<T>::above(v[g], k, e, lo_s[j])) bytes[k][e] |= 0xffffffffu << (ni * BITS);
          }
        }
        if (ni == WPT - 1) {
#pragma unroll
          for (int k = 0; k < CH; k++)
            Elem<T>::store_codes(packed + (sg0 + g / WPT) * GROUP + chunk_col<T>(k, i), bytes[k]);
        }
      }
      if ((g0 + ST) % WPT != 0) {
        // the codes of this stage exist before the next stage's loads are waited for
#pragma unroll
        for (int k = 0; k < CH; k++)
#pragma unroll
          for (int e = 0; e < W; e++) asm volatile("" : "+v"(bytes[k][e]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    return;
  }
#pragma unroll
  for (int g = 0; g < GPR; g++) {
    if (n0 + g < N) load_group<T>(x, numel, n0 + g, i, v[g]);
  }
#pragma unroll
  for (int g = 0; g < GPR; g++) {
    const int64_t n = n0 + g;
    lo_t[g] = (Stat)0.0f;
    hi_t[g] = (Stat)0.0f;
    if (n < N) {
      if (GIVEN) {
        lo_t[g] = Elem<T>::stat_of(mn_io[n]);
        hi_t[g] = Elem<T>::stat_of(mx_io[n]);
      } else {
        Elem<T>::group_minmax(v[g], lo_t[g], hi_t[g]);
      }
    }
  }
  // one scale division per lane: lane j of the row takes group j % GPR, then the row shares the results
  {
    const int mine = i & (GPR - 1);
    Stat lo_m = lo_t[0], hi_m = hi_t[0];
#pragma unroll
    for (int g = 1; g < GPR; g++) {
      lo_m = (mine == g) ? lo_t[g] : lo_m;
      hi_m = (mine == g) ? hi_t[g] : hi_m;
    }
    const Stat s_m = Elem<T>::make_scale(lo_m, hi_m, QMAX);
    if (i < GPR && n0 + i < N) {
      scale_out[n0 + i] = s_m;
      if (!GIVEN) {
        mn_io[n0 + i] = Elem<T>::elem_of(lo_m);
        if (mx_io) mx_io[n0 + i] = Elem<T>::elem_of(hi_m);
      }
    }
    if (GPR == 1) {
      s_t[0] = s_m;
    } else {
      s_t[0] = row_bcast<0>(s_m);
      if (GPR > 1) s_t[1 % GPR] = row_bcast<1>(s_m);
      if (GPR > 2) { s_t[2 % GPR] = row_bcast<2>(s_m); s_t[3 % GPR] = row_bcast<3>(s_m); }
      if (GPR > 4) {
        s_t[4 % GPR] = row_bcast<4>(s_m); s_t[5 % GPR] = row_bcast<5>(s_m);
        s_t[6 % GPR] = row_bcast<6>(s_m); s_t[7 % GPR] = row_bcast<7>(s_m);
      }
    }
  }

  FastRow<T, GPR> fast;
#pragma unroll
  for (int q = 0; q < SGR; q++) {
    const int64_t sg = sg0 + q;
    if (q == 0 || sg * WPT < N) {
    uint32_t bytes[CH][W];
#pragma unroll
    for (int k = 0; k < CH; k++)
#pragma unroll
      for (int e = 0; e < W; e++) bytes[k][e] = 0;

    if (NOISE == GACT_NOISE_REF) {
      // one Philox state per output byte j: key = seed, counter = (draw/4, 0, j lo, j hi); two neighbouring bytes at
      // a time, so that the half path can take its elements in pairs
      const float addend = uniform_addend();
#pragma unroll
      for (int k = 0; k < CH; k++)
#pragma unroll
        for (int e = 0; e < W; e += 2) {
          const uint64_t j = (uint64_t)sg * GROUP + chunk_col<T>(k, i) + e;
          uint32_t ra[4], rb[4];
#pragma unroll
          for (int ni = 0; ni < WPT; ni++) {
            const int g = q * WPT + ni;
            if ((ni & 3) == 0) {
              philox4x32<PHILOX_REF_ROUNDS>(ni >> 2, 0u, (uint32_t)j, (uint32_t)(j >> 32), k0, k1, ra);
              philox4x32<PHILOX_REF_ROUNDS>(ni >> 2, 0u, (uint32_t)(j + 1), (uint32_t)((j + 1) >> 32), k0, k1, rb);
            }
            if (n0 + g < N) {
              uint32_t ca, cb;
              Elem<T>::template code2<GIVEN>(v[g], k, e, lo_t[g], s_t[g], curand_uniform_map(ra[ni & 3], addend),
                                             curand_uniform_map(rb[ni & 3], addend), ca, cb);
              bytes[k][e] |= ca << (ni * BITS);
              bytes[k][e + 1] |= cb << (ni * BITS);
            }
          }
        }
    } else {
#pragma unroll
      for (int ni = 0; ni < WPT; ni++) {
        const int g = q * WPT + ni;
        const int64_t n = n0 + g;
        if (n < N) {
          if (NOISE == GACT_NOISE_FAST) {
            float cd[CH / 2][W];
            fast.draws(g, n0, i, k0, k1, cd);
#pragma unroll
            for (int k = 0; k < CH; k++) {
              uint32_t c[W];
              if (k < CH / 2) Elem<T>::template codes<false, GIVEN, true, false>(v[g], k, lo_t[g], s_t[g], cd[k % (CH / 2)], c);
              else Elem<T>::template codes<false, GIVEN, true, true>(v[g], k, lo_t[g], s_t[g], cd[k % (CH / 2)], c);
#pragma unroll
              for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << (ni * BITS);
            }
          } else {
            float u[CH][W];
#pragma unroll
            for (int k = 0; k < CH; k++) {
              if (NOISE == GACT_NOISE_INJECT) {
                Elem<T>::load_noise(noise + n * GROUP + chunk_col<T>(k, i), u[k]);
              } else {
#pragma unroll
                for (int e = 0; e < W; e++) u[k][e] = 0.5f;
              }
            }
#pragma unroll
            for (int k = 0; k < CH; k++) {
              uint32_t c[W];
              Elem<T>::template codes<NOISE == GACT_NOISE_CONST, GIVEN>(v[g], k, lo_t[g], s_t[g], u[k], c);
#pragma unroll
              for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << (ni * BITS);
            }
          }
        }
      }
    }

    if (Elem<T>::kRepairsInfiniteScale && !GIVEN) {
      // rare: a scale of the super-group overflowed to +inf (see Elem<T>::kRepairsInfiniteScale)
      bool any_inf = false;
#pragma unroll
      for (int ni = 0; ni < WPT; ni++) any_inf |= Elem<T>::scale_is_inf(s_t[q * WPT + ni]);
      if (__builtin_amdgcn_ballot_w64(any_inf) != 0) {
#pragma unroll
        for (int ni = 0; ni < WPT; ni++) {
          const int g = q * WPT + ni;
          if (n0 + g < N && Elem<T>::scale_is_inf(s_t[g])) {
#pragma unroll
            for (int k = 0; k < CH; k++)
#pragma unroll
              for (int e = 0; e < W; e++)
                if (Elem<T>::above(v[g], k, e, lo_t[g])) bytes[k][e] |= 0xffffffffu << (ni * BITS);
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < CH; k++) Elem<T>::store_codes(packed + sg * GROUP + chunk_col<T>(k, i), bytes[k]);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Dequantize a unit: G = SGS * (8/BITS) / PARTS consecutive groups - SGS whole super-groups, or (PARTS > 1, SGS = 1)
// one of PARTS equal parts of a super-group, the code words of which its other units load as well.  A lane owns the
// W = 16/sizeof(T) columns W*l .. W*l+W-1 of every group (one 16-byte store per group), so 256/W lanes cover a
// group: a whole wave per unit for float, half a wave for half.  All code words are loaded first, then the
// groups are written, each store instruction covering whole groups contiguously.
// The values follow quantization_cuda_kernel.cu:149-177: T(code) / scale with a real division, + min.
// 1, 2 and 4 bit tabulate the 2^BITS values of a group once and look them up; 8 bit computes
// them per element from one correctly rounded reciprocal per group.
// ------------------------------------------------------------------------------------------------
// value of lane g (0..7) of the row in every lane of the row; g is a constant once the caller's loop is unrolled
__device__ __forceinline__ float row_bcast_at(float v, int g) {
  switch (g) {
    case 0: return row_bcast<0>(v);
    case 1: return row_bcast<1>(v);
    case 2: return row_bcast<2>(v);
    case 3: return row_bcast<3>(v);
    case 4: return row_bcast<4>(v);
    case 5: return row_bcast<5>(v);
    case 6: return row_bcast<6>(v);
    default: return row_bcast<7>(v);
  }
}

template <typename T, int BITS, int SGS, int PARTS = 1, bool LARGE = true, bool SHARE_STATS = true>
__device__ __forceinline__ void dequantize_unit(const uint8_t* __restrict__ packed,
                                                const typename Elem<T>::Stat* __restrict__ scale,
                                                const T* __restrict__ mn, int64_t numel, int64_t N, int64_t unit,
                                                int l, T* __restrict__ out) {
  typedef typename Elem<T>::Stat Stat;
  constexpr int WPT = 8 / BITS;
  constexpr int W = Elem<T>::kDqWidth;
  constexpr int NI = WPT / PARTS;   // groups of a super-group that this unit writes
  constexpr int G = SGS * NI;
  static_assert(PARTS >= 1 && WPT % PARTS == 0 && (PARTS == 1 || SGS == 1), "parts divide one super-group");
  static_assert(G >= 1 && G <= ROW_GROUPS && (G & (G - 1)) == 0, "a dequantize unit is 1, 2, 4 or 8 groups");
  const int64_t sg0 = unit / PARTS * SGS;
  const int part = (int)(unit % PARTS);
  const int64_t n_sg = (N + WPT - 1) / WPT;
  const int64_t g0 = sg0 * WPT + part * NI;   // first group of the unit
  const int rl = l & 15;  // lane within its 16-lane row
  // float at 1 bit keeps the plain nontemporal store on large tensors (and in the batched launch)
  constexpr int POLICY = (sizeof(T) == 4 && BITS == 1 && LARGE) ? GACT_STORE_NT : GACT_STORE_NT_SYSTEM;
  // the wave's output window starts at the first group of its first unit (a wave holds one or two units, in order)
  const int64_t window_first = wave_first(g0) * GROUP;
  const OutWindow window(out + window_first, (numel - window_first) * (int64_t)sizeof(T));
  uint32_t w[SGS][W / 4];
#pragma unroll
  for (int it = 0; it < SGS; it++) {
    const uint8_t* p = packed + (sg0 + it) * GROUP + W * l;
    const bool live = sg0 + it < n_sg;
    if (W == 4) {
      w[it][0] = live ? stream_load(reinterpret_cast<const uint32_t*>(p)) : 0u;
    } else {
      u32x2 t = {0u, 0u};
      if (live) t = stream_load(reinterpret_cast<const u32x2*>(p));
      w[it][0] = t.x;
      w[it][W / 4 - 1] = t.y;
    }
    if (PARTS > 1) {   // this part's fields down to where part 0 has them (the shift is less than a byte)
#pragma unroll
      for (int k = 0; k < W / 4; k++) w[it][k] >>= part * NI * BITS;
    }
  }

  if constexpr (BITS <= 4) {
    // A group has only 2^BITS distinct outputs T(c)/scale + min: 8 * 2^BITS values for the unit.  Its lanes
    // tabulate them - entry e = group * 2^BITS + code in lane e % LPU, pass e / LPU, each with the real
    // division and the real sum - and every element then fetches its value from the lane that holds it
    // (ds_bpermute: the LDS crossbar, no LDS memory).  2 vector instructions per element instead of 6, and
    // one or two divisions per lane (four for half at 4 bit) instead of one per element.
    constexpr int LPU = GROUP / W;
    constexpr int ENT = 1 << BITS, TOT = G * ENT, PASSES = (TOT + LPU - 1) / LPU;
    // Scale and min of the unit's groups.  SHARE_STATS: lane j < G of the unit loads those of group g0 + j - one load
    // instruction each, a handful of lanes active - and the table entries fetch theirs across the unit.  Letting every
    // entry load its own (2 * PASSES instructions, all lanes active, for a fraction of a percent of the bytes) cost the
    // single-tensor kernel 7 % at half 4 bit (67 M elements 30.3 -> 28.2 us) and 4 % at half 2 bit (134 M: 50.5 -> 48.5);
    // with half units of 8 groups sharing loses instead (the batched launch when it had such units: 2 bit 683 -> 705 us,
    // 4 bit 757 -> 812 for 1.83 G elements), and float units, a whole wave each, are within 1 % either way.
    const uint32_t unitbase = (threadIdx.x & 63u) & ~(uint32_t)(LPU - 1);  // first lane of the unit within its wave
    uint32_t tab[PASSES];
    if constexpr (SHARE_STATS) {
      Stat s_mine = (Stat)1.0f, m_mine = (Stat)0.0f;
      if (l < G && g0 + l < N) {
        s_mine = scale[g0 + l];
        m_mine = Elem<T>::stat_of(mn[g0 + l]);
      }
      uint32_t s_bits, m_bits;
      if constexpr (sizeof(Stat) == 4) {
        s_bits = __builtin_bit_cast(uint32_t, s_mine);
        m_bits = __builtin_bit_cast(uint32_t, m_mine);
      } else {
        s_bits = (uint32_t)__builtin_bit_cast(uint16_t, s_mine);
        m_bits = (uint32_t)__builtin_bit_cast(uint16_t, m_mine);
      }
#pragma unroll
      for (int p = 0; p < PASSES; p++) {
        const int e = p * LPU + l;   // entries past the table (e >= TOT) wrap onto a lane of the unit and are never fetched
        const uint32_t src = (unitbase + (uint32_t)((e / ENT) & (G - 1))) << 2;
        const uint32_t sb = (uint32_t)__builtin_amdgcn_ds_bpermute((int)src, (int)s_bits);
        const uint32_t mb = (uint32_t)__builtin_amdgcn_ds_bpermute((int)src, (int)m_bits);
        Stat sv, mv;
        if constexpr (sizeof(Stat) == 4) {
          sv = __builtin_bit_cast(Stat, sb);
          mv = __builtin_bit_cast(Stat, mb);
        } else {
          sv = __builtin_bit_cast(Stat, (uint16_t)sb);
          mv = __builtin_bit_cast(Stat, (uint16_t)mb);
        }
        tab[p] = Elem<T>::table_entry((float)(e & (ENT - 1)), sv, mv);
      }
    } else {
#pragma unroll
      for (int p = 0; p < PASSES; p++) {
        const int e = p * LPU + l;
        const int64_t g = g0 + e / ENT;
        const bool live = e < TOT && g < N;
        tab[p] = Elem<T>::table_entry((float)(e & (ENT - 1)), live ? scale[g] : (Stat)1.0f,
                                      live ? Elem<T>::stat_of(mn[g]) : (Stat)0.0f);
      }
    }
#pragma unroll
    for (int it = 0; it < SGS; it++) {
#pragma unroll
      for (int ni = 0; ni < NI; ni++) {
        const int64_t n = g0 + it * WPT + ni;
        if (n < N) {
          const int g = it * NI + ni;
          const uint32_t base4 = (unitbase + (uint32_t)((g * ENT) % LPU)) << 2;
          T v[W];
#pragma unroll
          for (int e = 0; e < W; e++) {
            const uint32_t c = __builtin_amdgcn_ubfe(w[it][e >> 2], 8 * (e & 3) + ni * BITS, BITS);
            v[e] = Elem<T>::from_bits((uint32_t)__builtin_amdgcn_ds_bpermute((int)((c << 2) + base4), (int)tab[(g * ENT) / LPU]));
          }
          const int64_t at = n * GROUP + W * l;
          if (n * GROUP + GROUP <= numel) {
            Elem<T>::template store_dq<POLICY>(window, (uint32_t)((at - window_first) * (int64_t)sizeof(T)), v);
          } else {
#pragma unroll
            for (int e = 0; e < W; e++)
              if (at + e < numel) out[at + e] = v[e];
          }
        }
      }
    }
    return;
  } else {
  // 8 bit.  scale and min of the unit's groups: 16-byte loads when the whole unit exists and the arrays allow it
  constexpr int PERS = 16 / (int)sizeof(Stat), PERM = 16 / (int)sizeof(T);
  Stat sv[G], mv[G];
  if (G % PERS == 0 && G % PERM == 0 && g0 + G <= N &&
      ((reinterpret_cast<uintptr_t>(scale + g0) | reinterpret_cast<uintptr_t>(mn + g0)) & 15u) == 0) {
    typedef Stat svec __attribute__((ext_vector_type(PERS)));
    typedef T mvec __attribute__((ext_vector_type(PERM)));
#pragma unroll
    for (int c = 0; c < G / PERS; c++) {
      const svec a = *reinterpret_cast<const svec*>(scale + g0 + c * PERS);
#pragma unroll
      for (int e = 0; e < PERS; e++) sv[c * PERS + e] = a[e];
    }
#pragma unroll
    for (int c = 0; c < G / PERM; c++) {
      const mvec m = *reinterpret_cast<const mvec*>(mn + g0 + c * PERM);
#pragma unroll
      for (int e = 0; e < PERM; e++) mv[c * PERM + e] = Elem<T>::stat_of(m[e]);
    }
  } else {
#pragma unroll
    for (int g = 0; g < G; g++) {
      sv[g] = g0 + g < N ? scale[g0 + g] : (Stat)1.0f;
      mv[g] = g0 + g < N ? Elem<T>::stat_of(mn[g0 + g]) : (Stat)0.0f;
    }
  }
  // one correctly rounded reciprocal per group and row instead of one per group and lane: row lane j takes
  // group j % G and the row shares the results; when any scale of the wave is outside the range the
  // reciprocal form is valid for, the wave takes the plain division instead
  const int64_t gm = g0 + (rl & (G - 1));
  const float s_mine = gm < N ? (float)scale[gm] : 1.0f;
  const float r_mine = 1.0f / s_mine;
  const bool by_reciprocal = __builtin_amdgcn_ballot_w64(!reciprocal_safe(s_mine)) == 0;
#pragma unroll
  for (int it = 0; it < SGS; it++) {
    const int64_t n = sg0 + it;
    if (n < N) {
      T v[W];
      if (by_reciprocal) {
        const float sf = (float)sv[it], r = row_bcast_at(r_mine, it);
#pragma unroll
        for (int e = 0; e < W; e++) {
          const int c = (int)__builtin_amdgcn_ubfe(w[it][e >> 2], 8 * (e & 3), 8);
          v[e] = Elem<T>::finish(div_by_reciprocal((float)c, sf, r), mv[it]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < W; e++) {
          const int c = (int)__builtin_amdgcn_ubfe(w[it][e >> 2], 8 * (e & 3), 8);
          v[e] = Elem<T>::finish((float)c / (float)sv[it], mv[it]);
        }
      }
      const int64_t at = n * GROUP + W * l;
      if (n * GROUP + GROUP <= numel) {
        Elem<T>::template store_dq<POLICY>(window, (uint32_t)((at - window_first) * (int64_t)sizeof(T)), v);
      } else {
#pragma unroll
        for (int e = 0; e < W; e++)
          if (at + e < numel) out[at + e] = v[e];
      }
    }
  }
  }
}

// Batched launch: a block owns 128 consecutive groups of one tensor whatever the width, so the grid does
// not depend on the widths.  Quantize: each of the workgroup's 16 rows takes 8 consecutive groups - BITS
// super-groups - in one go: no loop, 16 KB (half) in flight per wave at every width, one scale division per
// lane and 8 groups.
#ifndef GACT_QB_STAGE
#define GACT_QB_STAGE 0 /* groups at a time in the batched quantize rows (0: all 8 at once) */
#endif
template <typename T, int BITS, int NOISE>
__device__ __forceinline__ void quantize_block128(const T* __restrict__ x, int64_t numel, int64_t N, int64_t lb,
                                                  uint8_t* __restrict__ packed,
                                                  typename Elem<T>::Stat* __restrict__ scale_out,
                                                  T* __restrict__ mn_out, uint64_t seed) {
  constexpr int WPT = 8 / BITS;
  const int row = threadIdx.x >> 4, i = threadIdx.x & 15;
  const int64_t sg0 = (lb * 16 + row) * BITS;
  if (NOISE == GACT_NOISE_REF) {
    // one Philox block per output byte: far too much code to lay out for 8 groups at once; super-group by super-group
#pragma unroll 1
    for (int q = 0; q < BITS; q++)
      if ((sg0 + q) * WPT < N)
        quantize_supergroup<T, BITS, NOISE, false, 1>(x, numel, N, sg0 + q, i, packed, scale_out, mn_out, (T*)nullptr,
                                                      (uint32_t)seed, (uint32_t)(seed >> 32), nullptr);
  } else if (sg0 * WPT < N) {
    quantize_supergroup<T, BITS, NOISE, false, BITS, GACT_QB_STAGE>(x, numel, N, sg0, i, packed, scale_out, mn_out, (T*)nullptr,
                                                                    (uint32_t)seed, (uint32_t)(seed >> 32), nullptr);
  }
}
// Dequantize: four workgroups share a block of 128 groups, 32 groups each - 4 units of 8 groups for float (a wave
// each), 8 units of 4 groups for half and bfloat16 (half a wave each; at 1 bit a unit is half a super-group and two
// units load the same code words): one unit per slot, several in a row per wave cost 10-20 %.  Half units of 4 groups
// with their scale and min shared across the unit are what the single-tensor kernel prefers on tensors of this size;
// against two workgroups per block and half units of 8 groups (120 half tensors, 1.83 G elements, all at one width):
// 2 bit 696 -> 677 us, 4 bit 758 -> 732, 8 bit 937 -> 929, 1 bit 651 -> 683; a mix of widths 719 -> 687.
template <typename T, int BITS>
__device__ __forceinline__ void dequantize_block128(const uint8_t* __restrict__ packed,
                                                    const typename Elem<T>::Stat* __restrict__ scale,
                                                    const T* __restrict__ mn, int64_t numel, int64_t N, int64_t lb,
                                                    int quarter, T* __restrict__ out) {
  constexpr int LPU = GROUP / Elem<T>::kDqWidth;  // lanes per unit
  constexpr int SLOTS = 256 / LPU;                // units of the workgroup
  const int slot = threadIdx.x / LPU, l = threadIdx.x % LPU;
  if constexpr (LPU == 64) {
    const int64_t unit = lb * 16 + quarter * SLOTS + slot;   // units of 8 groups
    if (unit * 8 < N) dequantize_unit<T, BITS, BITS, 1, true, false>(packed, scale, mn, numel, N, unit, l, out);
  } else {
    const int64_t unit = lb * 32 + quarter * SLOTS + slot;   // units of 4 groups
    constexpr int SGS = BITS == 1 ? 1 : BITS / 2, PARTS = BITS == 1 ? 2 : 1;
    if (unit * 4 < N) dequantize_unit<T, BITS, SGS, PARTS, true, true>(packed, scale, mn, numel, N, unit, l, out);
  }
}

// Row min/max only (the minimax entry point at D = 256): a 16-lane row takes MINIMAX_ROW_GROUPS consecutive
// groups, issues all their loads, reduces them one after the other and lets lane g store the results of group g.
// One group per row in one-wave workgroups (4 KB per float wave) reads fastest.  float, buffers cold in every cache,
// 1 group per row in 64-thread workgroups / 2 in 256 / 4 in 256 / 8 in 256: 4 M elements 4.68 / 4.81 / 5.44 / 5.94 us,
// 43 M 26.6 / 26.9 / 29.0 / 31.9, 103 M 60.3 / 61.6 / 61.8 / 65.6, 256 M 148.9 / 155.1 / 155.6 / 159; half 17 M
// 6.81 / 7.16 / 7.30 / 8.39, 256 M 72.3 / 74.8 / 75.7 / 77.7.
#define MINIMAX_ROW_GROUPS 1
#define MINIMAX_THREADS 64
template <typename T>
__device__ __forceinline__ void minimax_row(const T* __restrict__ x, int64_t N, int64_t row, int i,
                                            T* __restrict__ mn, T* __restrict__ mx) {
  const int64_t n0 = row * MINIMAX_ROW_GROUPS;
  typename Elem<T>::Store v[MINIMAX_ROW_GROUPS];
#pragma unroll
  for (int g = 0; g < MINIMAX_ROW_GROUPS; g++)
    if (n0 + g < N) load_group<T>(x, N * GROUP, n0 + g, i, v[g]);
  T lo_m = (T)0.0f, hi_m = (T)0.0f;
#pragma unroll
  for (int g = 0; g < MINIMAX_ROW_GROUPS; g++) {
    if (n0 + g < N) {
      T lo, hi;
      Elem<T>::group_minmax(v[g], lo, hi);
      lo_m = i == g ? lo : lo_m;
      hi_m = i == g ? hi : hi_m;
    }
  }
  if (i < MINIMAX_ROW_GROUPS && n0 + i < N) {
    mn[n0 + i] = lo_m;
    mx[n0 + i] = hi_m;
  }
}

// ------------------------------------------------------------------------------------------------
// Single-tensor kernels.
// ------------------------------------------------------------------------------------------------

// Workgroups go to the 8 XCDs round-robin (workgroup b runs on XCD b % 8) and every XCD streams through its
// own L2.  With the plain mapping an XCD sees every 8th tile, i.e. addresses in which three bits never
// change; handing each XCD runs of RUN consecutive tiles instead lets its writes leave as contiguous
// stretches (pure-write kernels with 8 KB per wave: 5.4 -> 6.2 TB/s).  The tail that does not fill a
// round of 8 * RUN tiles keeps the plain mapping.  RUN = 0 switches the remapping off.
#ifndef GACT_XCD_RUN_DQ
#define GACT_XCD_RUN_DQ 16
#endif
#ifndef GACT_XCD_RUN_DQB
#define GACT_XCD_RUN_DQB 16 /* batched dequantize */
#endif
#ifndef GACT_XCD_RUN_QB
#define GACT_XCD_RUN_QB 16 /* batched quantize: 4-6 % over the plain order at every width (120 half tensors, 1.83 G elements) */
#endif
#ifndef GACT_XCD_RUN_Q_LOW
#define GACT_XCD_RUN_Q_LOW 0 /* quantize, 1 bit: the long one-wave workgroups gain nothing or lose (mid-sized tensors 3 %) */
#endif
#ifndef GACT_XCD_RUN_Q
#define GACT_XCD_RUN_Q 128 /* quantize, 2, 4 and 8 bit: 2-6 % (half 2 bit 52.7 -> 50.2 us, float 2 bit 70.1 -> 68.8 us at 134 / 103 M elements) */
#endif
template <uint32_t RUN>
__device__ __forceinline__ uint32_t xcd_tile(uint32_t b, uint32_t nb) {
  if (RUN == 0) return b;
  constexpr uint32_t XCDS = 8, ROUND = XCDS * (RUN ? RUN : 1);
  if (b >= nb / ROUND * ROUND) return b;
  const uint32_t q = b / XCDS, x = b % XCDS;
  return ((q / (RUN ? RUN : 1)) * XCDS + x) * (RUN ? RUN : 1) + q % (RUN ? RUN : 1);
}

// The seed of a launch: a host value plus, optionally, a value read from device memory when the kernel runs -
// so that a launch recorded in a HIP graph draws fresh noise on every replay (the host updates the device word
// between replays).
struct SeedArg {
  uint64_t seed;
  const uint64_t* add;  // device pointer or null
  __device__ __forceinline__ uint64_t value() const { return add ? seed + *add : seed; }
};

// Geometry of the single-tensor quantize launch for an element type and width (1, 2, 4, 8 bit): super-groups per
// row (a row always issues the loads of all its groups first), threads per workgroup, the XCD-aware run of tiles,
// and how many groups at a time a row of whole groups is worked through (0: all at once) - `stage` in general,
// `stage_small` for tensors of fewer than `small_below` groups - with each stage issuing its own loads (`lazy`,
// `lazy_small`) instead of the row issuing all of them first.  Overridable at compile time
// (-DGACT_QGEOM_F32=..., _F16, _BF16) for experiments.
struct QGeom { int sgr, threads, run, stage, stage_small, small_below; bool lazy, lazy_small; };
#ifndef GACT_QGEOM_F16
#define GACT_QGEOM_F16 {{1, 64, 0, 4, 4, 1 << 15, true, false}, {1, 64, 128, 2, 2, 0, true, true}, {1, 64, 128, 1, 1, 0, true, true}, {1, 64, 128, 0, 0, 0, false, false}}
#endif
#ifndef GACT_QGEOM_BF16
#define GACT_QGEOM_BF16 {{1, 64, 0, 4, 4, 1 << 15, true, false}, {1, 64, 128, 2, 2, 0, true, true}, {1, 64, 128, 1, 1, 0, true, true}, {1, 64, 128, 0, 0, 0, false, false}}
#endif
// Staging pays where few waves share a SIMD and costs its extra divisions elsewhere.  float, quantize alone:
//   1 bit, 4 groups at a time: 8 M elements 9.8 -> 8.4 us, 17 M 14.5 -> 13.6, 34 M unchanged, 43 M 32.0 -> 32.4;
//   2 bit, group by group: 4 M 5.70 -> 5.51 us, 103 M 69.0 -> 67.8; two at a time is 2 % better still at 4 M and
//     1-2 % worse from 17 M on;  4 bit, group by group: 4 M 5.88 -> 5.73 us, unchanged at 103 M.
// half: 1 bit, 4 groups at a time: 4 M elements 6.7 -> 6.3 us, 17 M 11.8 -> 10.5, 67 M 29.0 -> 28.3;  2 bit, two at a
//   time: 2 % faster up to 17 M, 2 % slower at 67 M and 134 M (group by group: 3-8 % slower);  4 bit: within 1 %.
//   8 bit in one-wave workgroups: 4 M elements 4.78 -> 4.41 us, 17 M 10.7 -> 10.5, 67 M 32.3 -> 31.8 (4 bit and float 8 bit lose 1-5 % that way).
//   stages that issue their own loads: 1 bit 4 M elements 6.27 -> 6.67 us, 17 M 10.4 -> 10.1, 34 M 16.3 -> 15.9, 134 M 49.8 -> 49.0
//   (hence from 2^15 groups on);  2 bit, two at a time: 4 M unchanged, 17 M 10.0 -> 9.2, 26 M 13.8 -> 12.9, 134 M 51.0 -> 49.5,
//   256 M 93.0 -> 91.5 (bfloat16 67 M: 27.8 -> 26.4);  4 bit, group by group: 8 M 6.66 -> 6.3, 67 M and 256 M within 1 %.
//   float: 1 bit, four at a time: 4 M 6.5 -> 7.5 us, 17 M 13.6 -> 12.8, 103 M 69.3 -> 67.5, 256 M 170 -> 167 (from 2^15 groups on);
//   4 bit group by group: 4 M 5.64 -> 5.41, 8 M 8.29 -> 8.15, larger within 1 %;  2 bit within 2 % either way: not used.
#ifndef GACT_QGEOM_F32
#define GACT_QGEOM_F32 {{1, 64, 0, 4, 4, 1 << 15, true, false}, {1, 64, 128, 1, 2, 1 << 15, false, false}, {1, 64, 128, 1, 1, 0, true, true}, {1, 256, 128, 0, 0, 0, false, false}}
#endif
template <typename T>
__host__ __device__ constexpr QGeom q_geom(int bits) {
  constexpr QGeom f32[4] = GACT_QGEOM_F32, f16[4] = GACT_QGEOM_F16, b16[4] = GACT_QGEOM_BF16;
  const int k = bits == 1 ? 0 : bits == 2 ? 1 : bits == 4 ? 2 : 3;
  return Elem<T>::kDtype == GACT_F32 ? f32[k] : Elem<T>::kDtype == GACT_F16 ? f16[k] : b16[k];
}

// Geometry of the single-tensor dequantize launch for 1, 2, 4 and 8 bit: super-groups per unit, parts a
// super-group is split into (sgs = 1 then), threads per workgroup, XCD-aware run of tiles - and the same pair
// (sgs, parts) for large tensors (`large_from` groups and more), with the bytes of dynamic LDS a workgroup
// of 256 threads asks for from `cap_from` groups on without touching them (0: none; see the occupancy caps below).
// Units are 4 or 8 groups; units of 1 or 2 groups cost 10-150 %: every unit pays its code loads, its table and its
// divisions.  Dequantize alone, us, units of 4 against units of 8 (no cap), by groups in the tensor:
//   float 1 bit  65 536: 13.95 / 12.29   100 000: 20.0 / 18.4    (2 and 4 bit alike: 8)
//   float 8 bit  65 536: 15.76 / 15.98   100 000: 23.2 / 23.7    (4, and 8 with the cap from 2^17 groups)
//   half  1 bit  16 384: 3.86 / 4.36   65 536: 6.8 / 7.4   81 920: 10.3 / 8.8   98 304: 10.4 / 10.4   130 000: 14.2 / 13.3
//                (8 from 73 728 groups; capped at 6 workgroups per CU from 2^18 groups: 67 M elements 25.7 -> 24.8 us, 134 M
//                48.8 -> 46.7, 268 M 98.3 -> 90.4, while the same cap costs 6-12 % at 29-34 M; 2 and 4 bit lose 2-30 % by any cap)
//   half  2 bit  16 384: 3.87 / 4.73   65 536: 7.41 / 8.15   130 000: 14.5 / 13.8   1 M: 94.6 / 99.4   (4 throughout)
//   half  4 bit  16 384: 4.39 / 5.05   65 536: 8.08 / 8.95   200 000: 24.0 / 24.0   401 408: 45.0 / 46.7   1 M: 105.1 / 106.7
//   half  8 bit  65 536: 9.21 / 9.40   130 000: 18.0 / 18.2
struct DqGeom { int sgs, parts, threads, run, sgs_large, parts_large; unsigned lds_large; int large_from, cap_from; };
#ifndef GACT_DQGEOM_F32
#define GACT_DQGEOM_F32 {{1, 1, 256, GACT_XCD_RUN_DQ, 1, 1, 53000u, 1 << 17, 1 << 17}, {2, 1, 256, GACT_XCD_RUN_DQ, 2, 1, 53000u, 1 << 17, 1 << 17}, \
                         {4, 1, 256, GACT_XCD_RUN_DQ, 4, 1, 53000u, 1 << 17, 1 << 17}, {4, 1, 256, GACT_XCD_RUN_DQ, 8, 1, 53000u, 1 << 17, 1 << 17}}
#endif
#ifndef GACT_DQGEOM_F16
#define GACT_DQGEOM_F16 {{1, 2, 256, GACT_XCD_RUN_DQ, 1, 1, 26000u, 9 << 13, 1 << 18}, {1, 1, 256, GACT_XCD_RUN_DQ, 1, 1, 0u, 1 << 17, 1 << 17}, \
                         {2, 1, 256, GACT_XCD_RUN_DQ, 2, 1, 0u, 3 << 15, 3 << 15}, {4, 1, 256, GACT_XCD_RUN_DQ, 8, 1, 40000u, 1 << 17, 1 << 17}}
#endif
template <typename T>
__host__ __device__ constexpr DqGeom dq_geom(int bits) {
  constexpr DqGeom f32[4] = GACT_DQGEOM_F32, f16[4] = GACT_DQGEOM_F16;
  const int k = bits == 1 ? 0 : bits == 2 ? 1 : bits == 4 ? 2 : 3;
  return sizeof(T) == 4 ? f32[k] : f16[k];
}
__host__ __device__ constexpr int dq_unit_groups(DqGeom d, int bits, bool large) {
  return (large ? d.sgs_large : d.sgs) * (8 / bits) / (large ? d.parts_large : d.parts);
}

// The seed, a structure, comes first: the library is built with the kernels' leading scalar arguments preloaded into
// registers, which pays for dequantize and costs the quantize kernels up to 0.5 % - a structure is not preloaded,
// nor is anything behind it.
template <typename T, int BITS, int NOISE, bool GIVEN, bool SMALL = false>
__global__ void __launch_bounds__(256)
quantize_kernel(SeedArg seed_arg, const T* __restrict__ x, int64_t numel, int64_t N, uint8_t* __restrict__ packed,
                typename Elem<T>::Stat* __restrict__ scale_out, T* mn_io, T* mx_io, const float* __restrict__ noise) {
  constexpr QGeom G = q_geom<T>(BITS);
  constexpr int STAGE = SMALL ? G.stage_small : G.stage;
  constexpr bool LAZY = SMALL ? G.lazy_small : G.lazy;
  constexpr int SGR = NOISE == GACT_NOISE_REF ? 1 : G.sgr;   // the reference stream's code is too long to lay out several times
  // Tiles are handed out last first: the tensor's last tile - the only one that can be ragged, and then slower than
  // the others (169 343 float groups at 1 bit: 33.4 us when it is dispatched last, 31.6 when first) - goes to the
  // first workgroup instead of being the one the end of the kernel waits for.
  const uint32_t tile = gridDim.x - 1u - xcd_tile<(uint32_t)G.run>(blockIdx.x, gridDim.x);
  const int64_t sg0 = ((int64_t)tile * (blockDim.x >> 4) + (threadIdx.x >> 4)) * SGR;
  if (sg0 * (8 / BITS) >= N) return;
  const uint64_t seed = seed_arg.value();
  quantize_supergroup<T, BITS, NOISE, GIVEN, SGR, STAGE, LAZY>(x, numel, N, sg0, threadIdx.x & 15, packed, scale_out, mn_io, mx_io,
                                                  (uint32_t)seed, (uint32_t)(seed >> 32), noise);
}

// ------------------------------------------------------------------------------------------------
// Quantize at 1 bit with a wave per super-group: row r takes groups 2r and 2r + 1 of the 8 whose codes share bytes, the
// four rows OR their partial bytes together (two ds_bpermute steps on 4 dwords) and each then stores its quarter of the
// super-group's 256 bytes.  A wave holds 8 KB (float) or 4 KB (half) where a row per super-group makes it hold 32 or
// 16 KB and, with its 175 registers, leaves room for two waves per SIMD: 65 536 float groups are exactly one round of
// such waves, and the row form's time steps up with every further round (65 536 groups 12.9 us, 69 632: 16.2) where
// this form grows evenly (13.5, 14.4).  Float, us, row form / this form, by groups: 8 192: 5.3 / 4.8   32 768: 9.5 / 8.3
// 49 152: 11.3 / 10.8   57 344 .. 65 536: 11.8 .. 12.9 / 12.1 .. 13.5   73 728: 16.8 / 14.9   98 304: 19.7 / 19.4
// 131 072: 25.2 / 24.2   169 343: 31.4 / 30.7   229 376: 40.9 / 40.4   262 144 and more: equal.  Half: 8 192: 5.1 / 4.7
// 16 384: 5.4 / 4.6   32 768: 6.7 / 6.6   49 152: 8.2 / 8.3   65 536 and more: 9.2 / 9.9 .. 48.8 / 51.2.  At 2 bit (one
// group per row) there is nothing in it at any size.  Same results as quantize_kernel; not for the reference stream.
// ------------------------------------------------------------------------------------------------
#ifndef GACT_W8_RUN
#define GACT_W8_RUN 32
#endif
__device__ __forceinline__ uint32_t pack4(const uint32_t* b) {
  // the reference accumulates in a uint8_t: keep the low 8 bits of every byte
  return (b[0] & 0xffu) | ((b[1] & 0xffu) << 8) | ((b[2] & 0xffu) << 16) | (b[3] << 24);
}
template <typename T, int BITS, int NOISE>
__global__ void __launch_bounds__(256)
quantize_wave8_kernel(SeedArg seed_arg, const T* __restrict__ x, int64_t numel, int64_t N, uint8_t* __restrict__ packed,
                      typename Elem<T>::Stat* __restrict__ scale_out, T* __restrict__ mn_out, T* __restrict__ mx_out,
                      const float* __restrict__ noise) {
  static_assert(NOISE != GACT_NOISE_REF, "the reference stream draws per output byte");
  static_assert(BITS == 1 || BITS == 2, "four rows share a super-group: two groups a row at 1 bit, one at 2 bit");
  typedef typename Elem<T>::Stat Stat;
  constexpr int WPT = 8 / BITS, GR = WPT / 4, QMAX = (1 << BITS) - 1;   // GR: groups of a row
  constexpr int CH = Elem<T>::kQChunks, W = Elem<T>::kQWidth;
  const uint32_t tile = gridDim.x - 1u - xcd_tile<GACT_W8_RUN>(blockIdx.x, gridDim.x);   // last tile first, see quantize_kernel
  const int64_t sg = (int64_t)tile * (blockDim.x >> 6) + (threadIdx.x >> 6);               // the wave's super-group
  const int64_t n0 = sg * WPT;
  if (n0 >= N) return;   // the whole wave
  const int lane = threadIdx.x & 63, r = lane >> 4, i = lane & 15;
  const int64_t na = n0 + GR * r;   // the row's first group
  const uint64_t seed = seed_arg.value();
  const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);

  typename Elem<T>::Store v[GR];
#pragma unroll
  for (int g = 0; g < GR; g++)
    if (na + g < N) load_group<T>(x, numel, na + g, i, v[g]);
  Stat lo[GR], hi[GR], sc[GR];
#pragma unroll
  for (int g = 0; g < GR; g++) {
    lo[g] = hi[g] = (Stat)0.0f;
    if (na + g < N) Elem<T>::group_minmax(v[g], lo[g], hi[g]);
  }
  {
    const int mine = i & (GR - 1);   // with two groups a row, odd lanes divide for the second
    const Stat lo_m = mine ? lo[GR - 1] : lo[0], hi_m = mine ? hi[GR - 1] : hi[0];
    const Stat s_m = Elem<T>::make_scale(lo_m, hi_m, QMAX);
    if (i < GR && na + i < N) {
      scale_out[na + i] = s_m;
      mn_out[na + i] = Elem<T>::elem_of(lo_m);
      if (mx_out) mx_out[na + i] = Elem<T>::elem_of(hi_m);
    }
    sc[0] = GR == 1 ? s_m : row_bcast<0>(s_m);
    if (GR > 1) sc[GR - 1] = row_bcast<1>(s_m);
  }

  uint32_t bytes[CH][W];
#pragma unroll
  for (int k = 0; k < CH; k++)
#pragma unroll
    for (int e = 0; e < W; e++) bytes[k][e] = 0;
  FastRow<T, GR> fast;
#pragma unroll
  for (int g = 0; g < GR; g++) {
    const int64_t n = na + g;
    const uint32_t shift = (uint32_t)((GR * r + g) * BITS);   // the group's field within its bytes
    if (n < N) {
      if (NOISE == GACT_NOISE_FAST) {
        float cd[CH / 2][W];
        fast.draws(g, na, i, k0, k1, cd);
#pragma unroll
        for (int k = 0; k < CH; k++) {
          uint32_t c[W];
          if (k < CH / 2) Elem<T>::template codes<false, false, true, false>(v[g], k, lo[g], sc[g], cd[k % (CH / 2)], c);
          else Elem<T>::template codes<false, false, true, true>(v[g], k, lo[g], sc[g], cd[k % (CH / 2)], c);
#pragma unroll
          for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << shift;
        }
      } else {
#pragma unroll
        for (int k = 0; k < CH; k++) {
          float u[W];
          if (NOISE == GACT_NOISE_INJECT) {
            Elem<T>::load_noise(noise + n * GROUP + chunk_col<T>(k, i), u);
          } else {
#pragma unroll
            for (int e = 0; e < W; e++) u[e] = 0.5f;
          }
          uint32_t c[W];
          Elem<T>::template codes<NOISE == GACT_NOISE_CONST, false>(v[g], k, lo[g], sc[g], u, c);
#pragma unroll
          for (int e = 0; e < W; e++) bytes[k][e] |= c[e] << shift;
        }
      }
      if (Elem<T>::kRepairsInfiniteScale && Elem<T>::scale_is_inf(sc[g])) {   // rare, see Elem<T>::kRepairsInfiniteScale
#pragma unroll
        for (int k = 0; k < CH; k++)
#pragma unroll
          for (int e = 0; e < W; e++)
            if (Elem<T>::above(v[g], k, e, lo[g])) bytes[k][e] |= 0xffffffffu << shift;
      }
    }
  }

  // the lane's 16 bytes as 4 dwords in the order of their addresses, OR-ed over the four rows (every lane of the wave
  // is here: only whole waves left above)
  uint32_t pk[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    pk[j] = pack4(&bytes[j * 4 / W][(j * 4) % W]);
    pk[j] |= (uint32_t)__shfl_xor((int)pk[j], 16, 64);
    pk[j] |= (uint32_t)__shfl_xor((int)pk[j], 32, 64);
  }
  // row r stores dword r of every lane: float chunk r; half chunk r / 2, its columns 4 (r % 2) .. - 256 contiguous
  // bytes per store instruction either way
  const uint32_t mine = r == 0 ? pk[0] : r == 1 ? pk[1] : r == 2 ? pk[2] : pk[3];
  const int col = W == 4 ? chunk_col<T>(r, i) : chunk_col<T>(r >> 1, i) + 4 * (r & 1);
  stream_store(mine, reinterpret_cast<uint32_t*>(packed + sg * GROUP + col));
}

template <typename T, int BITS, bool LARGE = false>
__global__ void __launch_bounds__(256)
dequantize_kernel(const uint8_t* __restrict__ packed, const typename Elem<T>::Stat* __restrict__ scale,
                  const T* __restrict__ mn,
                  int64_t numel, int64_t N, T* __restrict__ out) {
  constexpr DqGeom D = dq_geom<T>(BITS);
  constexpr int LPU = GROUP / Elem<T>::kDqWidth;  // lanes per unit: 64 (float) or 32 (half)
  const int64_t unit = ((int64_t)xcd_tile<(uint32_t)D.run>(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x) / LPU;
  if (unit * dq_unit_groups(D, BITS, LARGE) >= N) return;
  dequantize_unit<T, BITS, LARGE ? D.sgs_large : D.sgs, LARGE ? D.parts_large : D.parts, LARGE>(packed, scale, mn, numel, N,
                                                                                              unit, threadIdx.x % LPU, out);
}

template <typename T>
__global__ void __launch_bounds__(256)
minimax256_kernel(const T* __restrict__ x, int64_t N, T* __restrict__ mn, T* __restrict__ mx) {
  const int64_t row = (int64_t)xcd_tile<GACT_XCD_RUN_Q>(blockIdx.x, gridDim.x) * (blockDim.x >> 4) + (threadIdx.x >> 4);
  if (row * MINIMAX_ROW_GROUPS >= N) return;
  minimax_row<T>(x, N, row, threadIdx.x & 15, mn, mx);
}

// ------------------------------------------------------------------------------------------------
// General shapes (any D for minimax; any G, D for pack / unpack).  These keep the operator surface
// complete; the path the library is built for is G = 1, D = 256 above.
// ------------------------------------------------------------------------------------------------
// Row min/max for any D.  2^lpr_log2 lanes share a row (8..64: as many as the row has 16-byte pieces, so
// short rows put several rows in a wave) and a lane group takes R consecutive rows, all of whose loads are
// issued before the first reduction.  VEC = false (a base address that is not 16-byte aligned) reads
// element by element.
template <typename T, bool VEC, int R>
__global__ void __launch_bounds__(256)
minimax_any_kernel(const T* __restrict__ x, int64_t N, int64_t D, int lpr_log2, T* __restrict__ mn,
                   T* __restrict__ mx) {
  constexpr int W = VEC ? 16 / (int)sizeof(T) : 1;
  typedef T vecw __attribute__((ext_vector_type(VEC ? W : 2)));
  typedef typename std::conditional<VEC, vecw, T>::type vec;
  const int lpr = 1 << lpr_log2;
  const int64_t group = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> lpr_log2;
  const int sub = threadIdx.x & (lpr - 1);
  const int64_t V = D / W;
  float lo[R], hi[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    lo[r] = Elem<T>::init_lo();
    hi[r] = Elem<T>::init_hi();
    const int64_t n = group * R + r;
    if (n < N) {
      const vec* row = reinterpret_cast<const vec*>(x + n * D);
#pragma unroll 4
      for (int64_t v = sub; v < V; v += lpr) {
        const vec q = stream_load(row + v);
#pragma unroll
        for (int e = 0; e < W; e++) {
          float f;
          if constexpr (VEC) f = (float)q[e]; else f = (float)q;
          lo[r] = __builtin_fminf(lo[r], f);
          hi[r] = __builtin_fmaxf(hi[r], f);
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
      if (off < lpr) {  // uniform over the launch
        lo[r] = __builtin_fminf(lo[r], __shfl_xor(lo[r], off, 64));
        hi[r] = __builtin_fmaxf(hi[r], __shfl_xor(hi[r], off, 64));
      }
    const int64_t n = group * R + r;
    if (sub == 0 && n < N) {
      mn[n] = Elem<T>::from_float(lo[r]);
      mx[n] = Elem<T>::from_float(hi[r]);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
scale_kernel(const T* __restrict__ mn, const T* __restrict__ mx, int bits, int64_t count, T* __restrict__ scale) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id < count) scale[id] = Elem<T>::make_scale(mn[id], mx[id], (1 << bits) - 1);
}

// one thread per output byte j = (no*G + g)*D + d
template <typename T, int NOISE>
__global__ void __launch_bounds__(256)
pack_any_kernel(const T* __restrict__ data, const T* __restrict__ mn, const T* __restrict__ scale, int bits,
                int64_t N, int64_t G, int64_t D, uint64_t seed, const float* __restrict__ noise,
                uint8_t* __restrict__ packed, int64_t total_bytes) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= total_bytes) return;
  const int wpt = 8 / bits;
  const int64_t d = j % D;
  const int64_t g = (j / D) % G;
  const int64_t no = j / (D * G);
  const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  uint32_t r[4];
  uint32_t byte = 0;
  for (int ni = 0; ni < wpt; ni++) {
    const int64_t n = no * wpt + ni;
    if (n >= N) break;
    const int64_t id = (n * G + g) * D + d;
    const int64_t sid = n * G + g;
    float u = 0.5f;
    if (NOISE == GACT_NOISE_INJECT) {
      u = noise[id];
    } else if (NOISE == GACT_NOISE_REF) {
      if ((ni & 3) == 0) philox4x32<PHILOX_REF_ROUNDS>(ni >> 2, 0u, (uint32_t)j, (uint32_t)((uint64_t)j >> 32), k0, k1, r);
      u = curand_uniform_map(r[ni & 3]);
    } else if (NOISE == GACT_NOISE_FAST) {
      const uint64_t blk = fast_block_of((uint64_t)id);
      philox4x32<PHILOX_FAST_ROUNDS>(0u, 0u, (uint32_t)blk, (uint32_t)(blk >> 32), k0, k1, r);
      u = fast_centred_of(r, (uint64_t)id);
    }
    typename Elem<T>::Store one;
    Elem<T>::set(one, 0, 0, data[id]);
    byte |= Elem<T>::template code1<true, NOISE == GACT_NOISE_FAST>(one, 0, 0, mn[sid], scale[sid], u) << (ni * bits);
  }
  packed[j] = (uint8_t)byte;
}

template <typename T>
__global__ void __launch_bounds__(256)
unpack_any_kernel(const uint8_t* __restrict__ packed, int bits, const T* __restrict__ scale,
                  const T* __restrict__ mn, int64_t N, int64_t G, int64_t D, T* __restrict__ out,
                  int64_t total_bytes) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= total_bytes) return;
  const int wpt = 8 / bits;
  const int64_t d = j % D;
  const int64_t g = (j / D) % G;
  const int64_t no = j / (D * G);
  const uint32_t byte = packed[j];
  for (int ni = 0; ni < wpt; ni++) {
    const int64_t n = no * wpt + ni;
    if (n >= N) break;
    const int64_t sid = n * G + g;
    int c = (int)((byte >> (ni * bits)) & ((1u << bits) - 1u));
    out[(n * G + g) * D + d] = Elem<T>::decode(c, Elem<T>::dq_prepare(scale[sid], mn[sid]));
  }
}

// G = 1 and D a multiple of 8 (every group size config.group_size can take): a thread owns 8 consecutive
// columns of one super-group - 8 output bytes, 8 elements of each of its 8/bits groups with 16-byte loads -
// and no thread divides 64-bit indices.  Same arithmetic and the same noise streams as pack_any_kernel.
template <typename T, int NOISE>
__global__ void __launch_bounds__(256)
pack_rows8_kernel(const T* __restrict__ data, const T* __restrict__ mn, const T* __restrict__ scale, int bits,
                  int64_t N, uint32_t tpr /* threads per super-group = D / 8 */, uint32_t total_threads, uint64_t seed,
                  const float* __restrict__ noise, uint8_t* __restrict__ packed) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total_threads) return;
  const int wpt = 8 / bits;
  const uint32_t no = t / tpr, c8 = t - no * tpr;
  const int64_t D = (int64_t)tpr * 8;
  const int64_t j0 = (int64_t)no * D + (int64_t)c8 * 8;  // first output byte
  const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  typedef T vec8 __attribute__((ext_vector_type(8)));
  uint32_t bytes[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  uint32_t r[8][4];
  for (int ni = 0; ni < wpt; ni++) {
    const int64_t n = (int64_t)no * wpt + ni;
    if (n >= N) break;
    const int64_t id0 = n * D + (int64_t)c8 * 8;
    const vec8 x = stream_load(reinterpret_cast<const vec8*>(data + id0));
    const T lo = mn[n], sc = scale[n];
    float u[8];
    if (NOISE == GACT_NOISE_INJECT) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(noise + id0), b = *reinterpret_cast<const f32x4*>(noise + id0 + 4);
      u[0] = a.x; u[1] = a.y; u[2] = a.z; u[3] = a.w; u[4] = b.x; u[5] = b.y; u[6] = b.z; u[7] = b.w;
    } else if (NOISE == GACT_NOISE_REF) {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const uint64_t j = (uint64_t)(j0 + e);
        if ((ni & 3) == 0) philox4x32<PHILOX_REF_ROUNDS>(ni >> 2, 0u, (uint32_t)j, (uint32_t)(j >> 32), k0, k1, r[e]);
        u[e] = curand_uniform_map(r[e][ni & 3]);
      }
    } else if (NOISE == GACT_NOISE_FAST) {
      // the thread's 8 consecutive elements share a block (id0 is a multiple of 8)
      const uint64_t blk = fast_block_of((uint64_t)id0);
      philox4x32<PHILOX_FAST_ROUNDS>(0u, 0u, (uint32_t)blk, (uint32_t)(blk >> 32), k0, k1, r[0]);
#pragma unroll
      for (int e = 0; e < 8; e++) u[e] = fast_centred_of(r[0], (uint64_t)id0 + e);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) u[e] = 0.5f;
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
      typename Elem<T>::Store one;
      Elem<T>::set(one, 0, 0, x[e]);
      bytes[e] |= Elem<T>::template code1<true, NOISE == GACT_NOISE_FAST>(one, 0, 0, lo, sc, u[e]) << (ni * bits);
    }
  }
  u32x2 w;
  w.x = (bytes[0] & 0xffu) | ((bytes[1] & 0xffu) << 8) | ((bytes[2] & 0xffu) << 16) | (bytes[3] << 24);
  w.y = (bytes[4] & 0xffu) | ((bytes[5] & 0xffu) << 8) | ((bytes[6] & 0xffu) << 16) | (bytes[7] << 24);
  stream_store(w, reinterpret_cast<u32x2*>(packed + j0));
}

template <typename T>
__global__ void __launch_bounds__(256)
unpack_rows8_kernel(const uint8_t* __restrict__ packed, int bits, const T* __restrict__ scale,
                    const T* __restrict__ mn, int64_t N, uint32_t tpr, uint32_t total_threads, T* __restrict__ out) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total_threads) return;
  const int wpt = 8 / bits;
  const uint32_t no = t / tpr, c8 = t - no * tpr;
  const int64_t D = (int64_t)tpr * 8;
  const u32x2 w = stream_load(reinterpret_cast<const u32x2*>(packed + (int64_t)no * D + (int64_t)c8 * 8));
  typedef T vec8 __attribute__((ext_vector_type(8)));
  for (int ni = 0; ni < wpt; ni++) {
    const int64_t n = (int64_t)no * wpt + ni;
    if (n >= N) break;
    const typename Elem<T>::Dq dq = Elem<T>::dq_prepare(scale[n], mn[n]);
    vec8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const uint32_t byte = ((e < 4 ? w.x : w.y) >> (8 * (e & 3))) & 0xffu;
      v[e] = Elem<T>::decode((int)((byte >> (ni * bits)) & ((1u << bits) - 1u)), dq);
    }
    stream_store(v, reinterpret_cast<vec8*>(out + n * D + (int64_t)c8 * 8));
  }
}

// ------------------------------------------------------------------------------------------------
// Dropout-mask bit packing.  Within each 512-element block, element e = k*16 + w is bit k of word w
// (quantization_cuda_kernel.cu:228-252): with one 16-byte load per lane, lane k holds elements
// 16k .. 16k+15, so word w is the ballot over lanes of "byte w is nonzero"; one wave packs two blocks
// (low and high half of each ballot).  A partial last block is packed sequentially (element e -> word
// e/32, bit e%32), which is the plain ballot of one byte per lane and fits the ceil(n/32)-word output.
// ------------------------------------------------------------------------------------------------
// A wave takes MASK_PAIRS consecutive pairs of blocks (4 KB of mask bytes) and issues all its loads first.
#ifndef MASK_PAIRS
#define MASK_PAIRS 4
#endif
__global__ void __launch_bounds__(256)
mask_pack_kernel(const uint8_t* __restrict__ data, int64_t n, int32_t* __restrict__ mask) {
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t full_blocks = n / 512;
  const int64_t pairs = (full_blocks + 1) / 2;
  const int64_t pair0 = wave * MASK_PAIRS;
  if (pair0 < pairs) {
    u32x4 q[MASK_PAIRS];
#pragma unroll
    for (int j = 0; j < MASK_PAIRS; j++) {
      const int64_t blk = (pair0 + j) * 2 + (lane >> 5);  // lanes 0..31 hold the pair's first block
      q[j] = u32x4{0u, 0u, 0u, 0u};
      if (blk < full_blocks) q[j] = stream_load(reinterpret_cast<const u32x4*>(data + (blk * 32 + (lane & 31)) * 16));
    }
    // word w of a block is the ballot of "byte w is nonzero" over the block's 32 lanes.  The 32 words of
    // pair j are collected in lanes 32 * (j & 1) ..: one store then writes two pairs.
    uint32_t mine[MASK_PAIRS / 2];
#pragma unroll
    for (int j = 0; j < MASK_PAIRS; j++) {
      uint32_t sel = 0;
#pragma unroll
      for (int w = 0; w < 16; w++) {
        const uint32_t word = w < 4 ? q[j].x : w < 8 ? q[j].y : w < 12 ? q[j].z : q[j].w;
        const uint64_t b = __ballot(((word >> (8 * (w & 3))) & 0xffu) != 0u);
        if ((lane & 15) == w) sel = (lane & 16) ? (uint32_t)(b >> 32) : (uint32_t)b;
      }
      if ((j & 1) == 0) mine[j >> 1] = sel;
      else if (lane >= 32) mine[j >> 1] = sel;
    }
#pragma unroll
    for (int jj = 0; jj < MASK_PAIRS / 2; jj++) {
      const int64_t word = (pair0 + 2 * jj) * 32 + lane;  // 16 words per block
      if ((word >> 4) < full_blocks) stream_store(mine[jj], reinterpret_cast<uint32_t*>(mask) + word);
    }
  }
  // the partial block goes to the wave after the last one that packs full blocks
  if (wave == (pairs + MASK_PAIRS - 1) / MASK_PAIRS) {
    const int64_t base = full_blocks * 512;
    const int64_t words = (n + 31) / 32;
    for (int64_t e0 = base; e0 < n; e0 += 64) {
      const int64_t e = e0 + lane;
      const uint64_t b = __ballot(e < n && data[e] != 0);
      const int64_t w = full_blocks * 16 + (e0 - base) / 32;
      if (lane == 0) mask[w] = (int32_t)(uint32_t)b;
      if (lane == 1 && w + 1 < words) mask[w + 1] = (int32_t)(uint32_t)(b >> 32);
    }
  }
}

// Unpack: a 16-lane row takes one block of 512 elements per step.  Lane r loads word r of the block (one
// 4-byte load, 64 contiguous bytes per row and 256 per wave), the row shares the 16 words by DPP broadcast,
// and lane r writes elements 16 r .. 16 r + 15 (bit r of every word) and 16 (r + 16) .. (bit r + 16): two 16-byte
// stores, each covering 256 contiguous bytes per row.  A wave takes MASK_STEPS steps (4 blocks each), all loads
// first.  (An earlier form let every lane load all 64 bytes of its block - 4 KB of requests per KB written: 75 us
// for 268 M elements against 47 us now, buffers cold in every cache.)
#ifndef MASK_STEPS
#define MASK_STEPS 2 /* 268 M elements: 49.1 us with 1, 47.4 with 2, 50.9 with 4, 55.2 with 8 */
#endif
template <int I>
__device__ __forceinline__ void mask_words_of_row(uint32_t mine, uint32_t (&w)[16]) {
  if constexpr (I < 16) {
    w[I] = row_bcast_u32<I>(mine);
    mask_words_of_row<I + 1>(mine, w);
  }
}
__global__ void __launch_bounds__(256)
mask_unpack_kernel(const int32_t* __restrict__ mask, int64_t n, uint8_t* __restrict__ out) {
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int row = lane >> 4, r = lane & 15;
  const int64_t full_blocks = n / 512;
  const int64_t blk0 = wave * (MASK_STEPS * 4);
  if (blk0 > full_blocks) return;
  // the wave's stores go through a window that starts at its first block (see OutWindow)
  const int64_t window_first = blk0 * 512;
  const OutWindow window(out + window_first, n - window_first);
  uint32_t mine[MASK_STEPS];
#pragma unroll
  for (int j = 0; j < MASK_STEPS; j++) {
    const int64_t blk = blk0 + j * 4 + row;
    mine[j] = blk < full_blocks ? (uint32_t)mask[blk * 16 + r] : 0u;
  }
#pragma unroll
  for (int j = 0; j < MASK_STEPS; j++) {
    const int64_t blk = blk0 + j * 4 + row;
    uint32_t w[16];
    mask_words_of_row<0>(mine[j], w);   // every lane of the wave takes part in the broadcasts
    if (blk < full_blocks) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int k = r + 16 * h;
        uint32_t q[4];
#pragma unroll
        for (int c = 0; c < 4; c++)
          q[c] = ((w[4 * c] >> k) & 1u) | (((w[4 * c + 1] >> k) & 1u) << 8) | (((w[4 * c + 2] >> k) & 1u) << 16) |
                 (((w[4 * c + 3] >> k) & 1u) << 24);
        window.store16<GACT_STORE_NT_SYSTEM>(u32x4{q[0], q[1], q[2], q[3]}, (uint32_t)((blk - blk0) * 512 + k * 16));
      }
    } else if (blk == full_blocks) {
      // the partial block, element by element: lane r of this row takes elements 32 r .. 32 r + 31
      const int64_t base = full_blocks * 512;
      for (int64_t e = base + r * 32; e < base + r * 32 + 32 && e < n; e++) {
        const int64_t rel = e - base;
        out[e] = (uint8_t)(((uint32_t)mask[full_blocks * 16 + rel / 32] >> (rel % 32)) & 1u);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Greedy bit allocation.  calc_precision.cc:66-118: a max-heap of (float key, index) compared
// lexicographically; indices are distinct, so the pop order is the descending total order and an
// argmax restates it.  Keys are doubles narrowed to float exactly as the heap's pair<float, int64> does.
// ------------------------------------------------------------------------------------------------
__host__ __device__ inline int prec_next_bits(int b) { return b == 32 ? 8 : b == 8 ? 4 : b == 4 ? 2 : b == 2 ? 1 : 0; }
__host__ __device__ inline float prec_key(float C, int b, int64_t w) {
  const int nb = prec_next_bits(b);
  const int coeff_2 = ((1 << nb) - 1) * ((1 << nb) - 1);
  double obj;
  if (b == 32) {
    obj = -(double)C / coeff_2;
  } else {
    const int coeff_1 = ((1 << b) - 1) * ((1 << b) - 1);
    obj = C * (1.0 / coeff_1 - 1.0 / coeff_2);
  }
  return (float)(obj / (double)(w * (int64_t)(b - nb)));
}
__host__ __device__ inline bool prec_valid_bits(int b) { return b == 1 || b == 2 || b == 4 || b == 8 || b == 32; }

#define PREC_MAX_L 4096      /* tensors the device kernel handles (LDS tables) */
#define PREC_SORT_MAX_L 4096 /* tensors the sorting path handles (4 candidate steps each, 8 bytes per candidate) */
#define PREC_THREADS 1024    /* largest workgroup the kernel is launched with */

// The sequential restatement of the heap loop by one wave: each step is a 64-lane argmax.  Used when a
// tensor's step keys do not decrease (never the case for the finite positive sensitivities the callers
// produce).
__device__ void calc_precision_sequential(int32_t* __restrict__ b_s, float* __restrict__ key_s,
                                          const float* __restrict__ C, const int64_t* __restrict__ w, int L,
                                          double b_sum, double target, int* rc_out) {
  const int lane = threadIdx.x;  // threadIdx.x < 64
  for (int idx = lane; idx < L; idx += 64)
    if (b_s[idx] > 1) key_s[idx] = prec_key(C[idx], b_s[idx], w[idx]);
  __builtin_amdgcn_wave_barrier();
  int rc = 0;
  while (b_sum > target) {
    float best_key = 0.0f;
    int best = -1;
    for (int idx = lane; idx < L; idx += 64) {
      if (b_s[idx] > 1) {
        const float k = key_s[idx];
        if (best < 0 || best_key < k || (!(k < best_key) && idx > best)) { best_key = k; best = idx; }
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float ok = __shfl_xor(best_key, off, 64);
      const int oi = __shfl_xor(best, off, 64);
      if (oi >= 0 && (best < 0 || best_key < ok || (!(ok < best_key) && oi > best))) { best_key = ok; best = oi; }
    }
    if (best < 0) { rc = GACT_EBUDGET; break; }
    const int cur = b_s[best];
    const int nb = prec_next_bits(cur);
    const int64_t wb = w[best];
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) {
      b_s[best] = nb;
      if (nb > 1) key_s[best] = prec_key(C[best], nb, wb);
    }
    b_sum -= (double)(wb * (int64_t)(cur - nb));
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  *rc_out = rc;
}

// order-preserving map of a float key to an unsigned integer (+0 and -0 compare equal in the heap)
__device__ __forceinline__ uint32_t sortable_key(float k) {
  if (k == 0.0f) k = 0.0f;
  const uint32_t u = __builtin_bit_cast(uint32_t, k);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Bitonic sort of M = R * NT candidate slots, descending, by a workgroup of NT threads (M and NT powers of two,
// NT >= 64).  Thread t keeps slots t, NT + t, ... in registers: partners NT or more apart are its own registers,
// partners less than a wave apart are reached with a shuffle, and only the passes in between go through LDS and
// a barrier (512 slots by 512 threads: 6 of 45 passes).
template <int R, int JR>
__device__ __forceinline__ void prec_exchange_own(uint64_t (&v)[R], int tid, int NT, int k) {
#pragma unroll
  for (int r = 0; r < R; r++) {
    if ((r & JR) == 0 && (r | JR) < R) {
      const bool descending = ((r * NT + tid) & k) == 0;
      const uint64_t a = v[r], b = v[r | JR];
      const uint64_t larger = a > b ? a : b, smaller = a > b ? b : a;
      v[r] = descending ? larger : smaller;   // slot r is the lower one of the pair
      v[r | JR] = descending ? smaller : larger;
    }
  }
}
template <int R>
__device__ __forceinline__ void prec_sort_slots(uint64_t* cand, int tid, int NT, int M) {
  uint64_t v[R];
#pragma unroll
  for (int r = 0; r < R; r++) v[r] = cand[r * NT + tid];
  for (int k = 2; k <= M; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      if (j >= NT) {
        switch (j / NT) {
          case 1: prec_exchange_own<R, 1>(v, tid, NT, k); break;
          case 2: prec_exchange_own<R, 2>(v, tid, NT, k); break;
          case 4: prec_exchange_own<R, 4>(v, tid, NT, k); break;
          default: prec_exchange_own<R, 8>(v, tid, NT, k); break;
        }
        continue;
      }
      uint64_t o[R];
      if (j >= 64) {
#pragma unroll
        for (int r = 0; r < R; r++) cand[r * NT + tid] = v[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; r++) o[r] = cand[(r * NT + tid) ^ j];
        __syncthreads();
      } else {
#pragma unroll
        for (int r = 0; r < R; r++) {
          const uint32_t lo32 = (uint32_t)__shfl_xor((int)(uint32_t)v[r], j, 64);
          const uint32_t hi32 = (uint32_t)__shfl_xor((int)(uint32_t)(v[r] >> 32), j, 64);
          o[r] = ((uint64_t)hi32 << 32) | lo32;
        }
      }
      // the lower slot of a pair keeps the larger key where the run descends, the smaller where it ascends
      const bool lower = (tid & j) == 0;
#pragma unroll
      for (int r = 0; r < R; r++) {
        const bool descending = ((r * NT + tid) & k) == 0;
        const uint64_t larger = v[r] > o[r] ? v[r] : o[r], smaller = v[r] > o[r] ? o[r] : v[r];
        v[r] = (descending == lower) ? larger : smaller;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++) cand[r * NT + tid] = v[r];
  __syncthreads();
}

// The greedy pops candidates (tensor i, step s) in descending (key, i) order.  A tensor's steps have
// strictly decreasing keys, so that order is the descending sort of ALL candidate steps by
// (key, index, earlier step first); the loop `while (b_sum > target) pop` then takes a prefix of it.
// One workgroup, one thread per candidate slot up to 1024: build up to 4 candidates per tensor, bitonic-sort them,
// prefix-sum the savings (integers, exact in double), apply the prefix.  Falls back to the sequential
// loop when that order argument does not hold.
__global__ void __launch_bounds__(PREC_THREADS)
calc_precision_kernel(int32_t* __restrict__ b, const float* __restrict__ C, const int64_t* __restrict__ w,
                      int L, double target, int32_t* __restrict__ status) {
  // dynamic LDS: one 8-byte slot per candidate, 4 per tensor rounded up to a power of two (128 KB for 4096
  // tensors); the sequential path reuses it for its float keys
  extern __shared__ uint64_t cand[];
  __shared__ int32_t b_s[PREC_MAX_L];
  __shared__ double part_s[PREC_THREADS];
  __shared__ int flag_s;
  const int tid = threadIdx.x, NT = blockDim.x;
  const bool sortable = L <= PREC_SORT_MAX_L;
  int M = 4;
  while (M < 4 * L) M <<= 1;
  if (tid == 0) flag_s = 0;
  if (sortable)
    for (int t = tid; t < M; t += NT) cand[t] = 0;  // 0 sorts after every real candidate
  __syncthreads();

  double part = 0.0;
  bool bad_order = false, bad_width = false;
  for (int idx = tid; idx < L; idx += NT) {
    const int bi = b[idx];
    b_s[idx] = bi;
    if (!prec_valid_bits(bi)) {
      bad_width = true;
    } else if (bi > 1) {
      const int64_t wi = w[idx];
      part += (double)((int64_t)bi * wi);
      if (sortable) {
        const float Ci = C[idx];
        float prev = __builtin_inff();
        int cur = bi, st = 0;
        while (cur > 1 && st < 4) {
          const float k = prec_key(Ci, cur, wi);
          if (!(k < prev) && !(k == prev && k == 0.0f)) bad_order = true;  // also catches NaN
          cand[idx * 4 + st] = ((uint64_t)sortable_key(k) << 32) | ((uint32_t)idx << 2) | (uint32_t)(3 - st);
          prev = k;
          cur = prec_next_bits(cur);
          st++;
        }
        if (cur > 1) bad_order = true;  // a width the 4-step descent does not know
      }
    }
  }
  part_s[tid] = part;
  if (bad_order) flag_s = 1;
  __syncthreads();
  if (bad_width) flag_s = 3;
  __syncthreads();
  if (flag_s == 3) {  // a width outside {1,2,4,8,32}: leave b as it is
    if (status && tid == 0) *status = GACT_EINVAL;
    return;
  }
  // every term is an integer; the sum is exact (and order-free) below 2^53
  for (int off = NT >> 1; off >= 1; off >>= 1) {
    if (tid < off) part_s[tid] += part_s[tid + off];
    __syncthreads();
  }
  const double b_sum0 = part_s[0];
  const bool sequential = !sortable || flag_s != 0;
  __syncthreads();

  int rc = 0;
  if (sequential) {
    if (tid < 64) calc_precision_sequential(b_s, reinterpret_cast<float*>(cand), C, w, L, b_sum0, target, &rc);
  } else {
    // bitonic sort, descending
    switch (M / NT) {
      case 1: prec_sort_slots<1>(cand, tid, NT, M); break;
      case 2: prec_sort_slots<2>(cand, tid, NT, M); break;
      case 4: prec_sort_slots<4>(cand, tid, NT, M); break;
      case 8: prec_sort_slots<8>(cand, tid, NT, M); break;
      default: prec_sort_slots<16>(cand, tid, NT, M); break;
    }
    // savings of the sorted candidates, chunked over the threads
    const int per = M / NT > 0 ? M / NT : 1;
    const int lo = tid * per, hi = lo + per < M ? lo + per : M;
    double mine = 0.0;
    for (int t = lo; t < hi && t < M; t++) {
      const uint64_t c = cand[t];
      if (c == 0) break;
      const int idx = (int)((uint32_t)c >> 2), st = 3 - (int)(c & 3u);
      int cur = b[idx];
      for (int q = 0; q < st; q++) cur = prec_next_bits(cur);
      mine += (double)(w[idx] * (int64_t)(cur - prec_next_bits(cur)));
    }
    // exclusive prefix of the threads' savings: a scan inside every wave, then the waves' totals (the terms are
    // integers below 2^53, so the sums are exact in any order)
    if (lo >= M) mine = 0.0;
    double incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const double up = __shfl_up(incl, off, 64);
      if ((tid & 63) >= off) incl += up;
    }
    if ((tid & 63) == 63) part_s[tid >> 6] = incl;   // at most 16 waves
    __syncthreads();
    double before = 0.0, total = 0.0;
    for (int wv = 0; wv < (NT + 63) >> 6; wv++) {
      const double v = part_s[wv];
      if (wv < (tid >> 6)) before += v;
      total += v;
    }
    if (tid == 0 && b_sum0 - total > target) flag_s = 2;  // every step taken and still over budget
    __syncthreads();
    double running = b_sum0 - (before + incl - mine);
    for (int t = lo; t < hi && t < M; t++) {
      const uint64_t c = cand[t];
      if (c == 0 || !(running > target)) break;
      const int idx = (int)((uint32_t)c >> 2), st = 3 - (int)(c & 3u);
      int cur = b[idx];
      for (int q = 0; q < st; q++) cur = prec_next_bits(cur);
      const int nb = prec_next_bits(cur);
      atomicMin(&b_s[idx], nb);
      running -= (double)(w[idx] * (int64_t)(cur - nb));
    }
    __syncthreads();
    if (flag_s == 2) rc = GACT_EBUDGET;
  }
  __syncthreads();
  for (int idx = tid; idx < L; idx += NT) b[idx] = b_s[idx];
  if (status && tid == 0) *status = rc;
}

// ------------------------------------------------------------------------------------------------
// Batched launch over a table of tensors with device-resident bits.
// ------------------------------------------------------------------------------------------------
// The workspace of a batched launch (device memory the caller brings, or the library's static array):
//   BatchHeader                      what the plan found
//   int32 block_tensor[total_blocks] tensor of every block of the grid
struct BatchHeader {
  int64_t need;            // arena bytes the table needs
  int64_t ok;              // 1: every width and element type valid and need <= capacity
  int64_t tensors_at[4];   // tensors at width 1, 2, 4, 8
  int64_t reserved[26];
};
static_assert(sizeof(BatchHeader) == 256, "the header is 32 int64");
struct BatchWorkspace {
  BatchHeader* hdr;
  int32_t* block_tensor;
};
__host__ __device__ inline int64_t batch_workspace_need(int64_t L, int64_t total_blocks) {
  (void)L;
  return (int64_t)sizeof(BatchHeader) + (total_blocks + 3) / 4 * 16;
}
__host__ __device__ inline BatchWorkspace batch_workspace(void* base) {
  BatchWorkspace w;
  w.hdr = (BatchHeader*)base;
  w.block_tensor = (int32_t*)((uint8_t*)base + sizeof(BatchHeader));
  return w;
}
__device__ __forceinline__ int width_index(int bits) { return bits == 1 ? 0 : bits == 2 ? 1 : bits == 4 ? 2 : 3; }

__device__ __forceinline__ int batch_find(const gact_batch_entry* __restrict__ table, int L, int64_t block) {
  int lo = 0, hi = L - 1;  // last entry with first_block <= block
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].first_block <= block) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The plan, one launch.  Workgroup 0 (its first wave): lane l sizes tensors l, l+64, ...; the running packed-arena
// offset is carried across rounds of 64 with a wave-wide inclusive scan.  The other workgroups, one thread per
// block of the grid: find the block's tensor and note it, so that a work kernel's block needs one load for it
// (this part depends on the geometry only, not on the widths).
__global__ void __launch_bounds__(256)
batch_plan_kernel(gact_batch_entry* table, const int32_t* __restrict__ bits, int L, int64_t total_blocks,
                  int64_t capacity, BatchWorkspace ws, int64_t* __restrict__ verdict) {
  if (blockIdx.x > 0) {
    const int64_t g = (int64_t)(blockIdx.x - 1) * blockDim.x + threadIdx.x;
    if (g < total_blocks) ws.block_tensor[g] = batch_find(table, L, g);
    return;
  }
  if (threadIdx.x >= 64) return;
  const int lane = threadIdx.x;
  int64_t base = 0;
  int bad = 0;
  int cnt[4] = {0, 0, 0, 0};
  for (int t0 = 0; t0 < L; t0 += 64) {
    const int t = t0 + lane;
    int64_t bytes = 0;
    if (t < L) {
      int bt = bits[t];
      if (!(bt == 1 || bt == 2 || bt == 4 || bt == 8)) { bad = 1; bt = 8; }
      const int dt = table[t].dtype;
      if (dt < 0 || dt > 2) bad = 1;
      cnt[width_index(bt)]++;
      const int wpt = 8 / bt;
      const int64_t N = (table[t].numel + GROUP - 1) / GROUP;
      const int64_t n_round = (N + wpt - 1) / wpt * wpt;
      bytes = ((int64_t)bt * n_round * (GROUP / 8) + 255) / 256 * 256;
    }
    int64_t incl = bytes;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int64_t up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    if (t < L) table[t].packed_offset = base + incl - bytes;
    base += __shfl(incl, 63, 64);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    bad |= __shfl_xor(bad, off, 64);
#pragma unroll
    for (int k = 0; k < 4; k++) cnt[k] += __shfl_xor(cnt[k], off, 64);
  }
  if (lane == 0) {
    const int64_t ok = (!bad && base <= capacity) ? 1 : 0;
    ws.hdr->need = base;
    ws.hdr->ok = ok;
    if (verdict) {   // the same two words where the caller can see them
      verdict[0] = base;
      verdict[1] = ok;
    }
#pragma unroll
    for (int k = 0; k < 4; k++) ws.hdr->tensors_at[k] = cnt[k];
  }
}

// Quantize, one launch per element type over all blocks of the grid: the width of a block's tensor is read from
// device memory and selects the code path (a row takes 8 groups whatever the width, so every path holds the same
// amount of data in registers); blocks of tensors of another element type leave at once.
template <typename T, int NOISE>
__global__ void __launch_bounds__(256)
quantize_batched_kernel(const gact_batch_entry* __restrict__ table, const int32_t* __restrict__ bits,
                        BatchWorkspace ws, uint8_t* __restrict__ packed_arena, uint8_t* __restrict__ scale_arena,
                        uint8_t* __restrict__ min_arena) {
  if (ws.hdr->ok == 0) return;  // the plan did not fit the arena or held an invalid width
  const int64_t block = xcd_tile<GACT_XCD_RUN_QB>(blockIdx.x, gridDim.x);
  const int t = ws.block_tensor[block];
  const gact_batch_entry ent = table[t];
  if (ent.dtype != Elem<T>::kDtype) return;
  const int64_t N = (ent.numel + GROUP - 1) / GROUP;
  const int64_t lb = block - ent.first_block;
  const T* x = (const T*)ent.x;
  uint8_t* packed = packed_arena + ent.packed_offset;
  typename Elem<T>::Stat* sc = (typename Elem<T>::Stat*)(scale_arena + ent.stats_offset * 4);
  T* mn = (T*)(min_arena + ent.stats_offset * 4);
  switch (bits[t]) {
    case 1: quantize_block128<T, 1, NOISE>(x, ent.numel, N, lb, packed, sc, mn, ent.seed); break;
    case 2: quantize_block128<T, 2, NOISE>(x, ent.numel, N, lb, packed, sc, mn, ent.seed); break;
    case 4: quantize_block128<T, 4, NOISE>(x, ent.numel, N, lb, packed, sc, mn, ent.seed); break;
    default: quantize_block128<T, 8, NOISE>(x, ent.numel, N, lb, packed, sc, mn, ent.seed); break;
  }
}

// Dequantize, one launch for all widths (every width fits 60 registers): the width of a block's tensor is read
// from device memory and selects the code path, so no workgroup is launched only to leave.
template <int BITS>
__device__ __forceinline__ void dequantize_batched_block(const gact_batch_entry& ent, int64_t lb, int quarter,
                                                         const uint8_t* packed, const uint8_t* sc, const uint8_t* mn) {
  const int64_t N = (ent.numel + GROUP - 1) / GROUP;
  if (ent.dtype == GACT_F32)
    dequantize_block128<float, BITS>(packed, (const float*)sc, (const float*)mn, ent.numel, N, lb, quarter, (float*)ent.x);
  else if (ent.dtype == GACT_F16)
    dequantize_block128<f16, BITS>(packed, (const f16*)sc, (const f16*)mn, ent.numel, N, lb, quarter, (f16*)ent.x);
  else
    dequantize_block128<bf16, BITS>(packed, (const float*)sc, (const bf16*)mn, ent.numel, N, lb, quarter, (bf16*)ent.x);
}
// grid: four workgroups per block of 128 groups
__global__ void __launch_bounds__(256)
dequantize_batched_kernel(const gact_batch_entry* __restrict__ table, const int32_t* __restrict__ bits,
                          BatchWorkspace ws, const uint8_t* __restrict__ packed_arena,
                          const uint8_t* __restrict__ scale_arena, const uint8_t* __restrict__ min_arena) {
  if (ws.hdr->ok == 0) return;
  // the XCD-aware order of the single-tensor kernel (715 -> 709 us on 120 half tensors)
  const uint32_t tile = xcd_tile<GACT_XCD_RUN_DQB>(blockIdx.x, gridDim.x);
  const int64_t block = tile >> 2;
  const int quarter = tile & 3;   // which quarter of the block
  const int t = ws.block_tensor[block];
  const gact_batch_entry ent = table[t];
  const int64_t lb = block - ent.first_block;
  const uint8_t* packed = packed_arena + ent.packed_offset;
  const uint8_t* sc = scale_arena + ent.stats_offset * 4;
  const uint8_t* mn = min_arena + ent.stats_offset * 4;
  switch (bits[t]) {
    case 1: dequantize_batched_block<1>(ent, lb, quarter, packed, sc, mn); break;
    case 2: dequantize_batched_block<2>(ent, lb, quarter, packed, sc, mn); break;
    case 4: dequantize_batched_block<4>(ent, lb, quarter, packed, sc, mn); break;
    default: dequantize_batched_block<8>(ent, lb, quarter, packed, sc, mn); break;
  }
}

// ------------------------------------------------------------------------------------------------
// Host side of the C ABI.
// ------------------------------------------------------------------------------------------------
namespace {

inline bool valid_bits(int bits) { return bits == 1 || bits == 2 || bits == 4 || bits == 8; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// hipGetLastError returns and clears the thread's last error, which may be one an earlier call of the caller's left
// behind: an entry point clears it before its first launch (fresh_launch) and reports what its own launches left.
inline void fresh_launch() { (void)hipGetLastError(); }
inline int launch_status() { return hipGetLastError() == hipSuccess ? GACT_OK : GACT_ELAUNCH; }

// one 16-lane row per unit of work (a super-group for quantize / dequantize, 8 groups for minimax);
// 16 rows per 256-thread block
inline void row_grid(int64_t rows, dim3* grid, dim3* block, int threads = 256) {
  const int rows_per_block = threads / 16;
  *grid = dim3((unsigned)((rows + rows_per_block - 1) / rows_per_block));
  *block = dim3(threads);
}
inline int64_t supergroups(int64_t N, int bits) { return (N + 8 / bits - 1) / (8 / bits); }

// Fewer resident waves per CU for some kernels on large tensors.  These streams mix a minority of traffic in
// the other direction into their main direction, and past a point more requests in flight make that mix more
// expensive for the memory system, not cheaper (a stand-alone kernel that writes 8 KB and reads 1 KB per
// wave: 88 us for 411 MB at full occupancy, 70 us at 2 waves per SIMD).  The cap is a request for dynamic
// LDS that the kernels never touch - a CU has 160 KB of it, so 53 000 bytes admit 3 workgroups.  What counts is
// the bytes in flight per CU: the cap goes with units of 8 groups (8 KB of stores per float wave); with units of 4
// it starves the CU (float 1 bit, 103 M elements: 66 us with units of 8 and the cap, 71 with units of 4 and no cap,
// 98 with units of 4 and the cap; float 8 bit: 80, 82, 96; half 8 bit, 256 M elements, 4 workgroups per CU: 119, 129,
// 147).  Hence the geometry table's own entries for large tensors.
// Interleaved A/B in both orders on a 411 MB float tensor (us, full occupancy -> capped), units of 8 groups:
// dequantize with 3 workgroups of 4 waves per CU 1 bit 76.3 -> 66.1, 2 bit 76.4 -> 69.6, 4 bit 77.6 -> 74.5,
// 8 bit 81.7 -> 79.9; quantize float 4 bit with 16 one-wave workgroups 76.1 -> 71.1.
// The other kernels (all half quantize, float quantize at 1, 2 and 8 bit) and small tensors gain nothing or
// lose, and keep full occupancy.
// From 2^17 groups (34 M elements) on (`large_from` in the geometry table): with buffers that are cold in every cache
// the cap costs 3-12 % at 8-26 M elements, is neutral at 31-34 M and gains 1-7 % from 43 M, 3-13 % at 84 M.
// Quantize, float: 4 bit capped at 16 one-wave workgroups per CU from 98 304 groups on (100 000 groups: 21.1 -> 20.9 us,
// 200 000: 40.1 -> 37.9, 401 408: 77.4 -> 72.6, 1 M: 191.5 -> 177.8; 65 536: 14.6 -> 14.65), 2 bit at 8 from 196 608 groups on
// (262 144 groups: 47.6 -> 46.2 us, 401 408: 72.2 -> 69.1, 1 M: 177.3 -> 165.3; 131 072: 25.3 -> 26.1).  Buffers cold in
// every cache.  1 and 8 bit gain 1-2 % at most, half loses at 4 and 8 bit and gains 1-2 % at 1 and 2 bit: left alone.
#ifndef GACT_QCAP_FROM_GROUPS
#define GACT_QCAP_FROM_GROUPS (3 << 15)
#endif
#ifndef GACT_QCAP2_FROM_GROUPS
#define GACT_QCAP2_FROM_GROUPS (3 << 16)
#endif
inline unsigned quantize_lds_cap(size_t elem_size, int bits, int64_t N) {
  if (elem_size != 4) return 0u;
  if (bits == 4) return N >= GACT_QCAP_FROM_GROUPS ? 10000u : 0u;
  if (bits == 2) return N >= GACT_QCAP2_FROM_GROUPS ? 20000u : 0u;
  return 0u;
}

// Below how many groups a 1-bit quantize takes the wave-per-super-group kernel (0: never), by element size.  (The kernel
// also exists at 2 bit - four rows of one group each, 4 KB per float wave - and is not launched there: float [4096,1024]
// at 2 bit, deterministic, 5.22 us with a row per super-group against 5.37-5.52 us that way, in workgroups of one or
// four waves, with or without the XCD-aware tile order; 13 M elements 11.3 against 11.4-11.8 us; 103 M 68.1 / 67.6-68.8.)
#ifndef GACT_W8_BELOW_F32
#define GACT_W8_BELOW_F32 (1 << 18)
#endif
#ifndef GACT_W8_BELOW_F16
#define GACT_W8_BELOW_F16 40960
#endif
#ifndef GACT_W8_THREADS
#define GACT_W8_THREADS 256
#endif

// What a single-tensor launch is made of: the kernel, its grid, and the dynamic LDS it asks for.  Planning and
// launching are separate so that gact_launch_geometry reports exactly what a launch would use.
struct LaunchPlan {
  const void* kernel = nullptr;   // null: the arguments name no kernel (an unknown noise mode or width)
  dim3 grid, block;
  unsigned lds = 0;
};

// the quantize kernel of a noise mode: its small-tensor form where the geometry has one (staging is for fused
// min/max and not for the reference stream)
template <typename T, int BITS, int NOISE, bool GIVEN>
const void* quantize_kernel_of(bool small) {
  constexpr QGeom G = q_geom<T>(BITS);
  if constexpr (!GIVEN && NOISE != GACT_NOISE_REF && (G.stage_small != G.stage || G.lazy_small != G.lazy)) {
    if (small) return (const void*)quantize_kernel<T, BITS, NOISE, GIVEN, true>;
  }
  return (const void*)quantize_kernel<T, BITS, NOISE, GIVEN, false>;
}

template <typename T, int BITS, bool GIVEN>
LaunchPlan plan_quantize(int64_t N, int noise_mode) {
  LaunchPlan p;
  constexpr QGeom G = q_geom<T>(BITS);
  if constexpr (!GIVEN && BITS == 1) {
    if (noise_mode != GACT_NOISE_REF && N < (sizeof(T) == 4 ? GACT_W8_BELOW_F32 : GACT_W8_BELOW_F16)) {
      const unsigned per_block = GACT_W8_THREADS / 64;
      p.grid = dim3((unsigned)((supergroups(N, BITS) + per_block - 1) / per_block));
      p.block = dim3(GACT_W8_THREADS);
      switch (noise_mode) {
        case GACT_NOISE_CONST: p.kernel = (const void*)quantize_wave8_kernel<T, BITS, GACT_NOISE_CONST>; break;
        case GACT_NOISE_INJECT: p.kernel = (const void*)quantize_wave8_kernel<T, BITS, GACT_NOISE_INJECT>; break;
        case GACT_NOISE_FAST: p.kernel = (const void*)quantize_wave8_kernel<T, BITS, GACT_NOISE_FAST>; break;
      }
      return p;
    }
  }
  const int sgr = noise_mode == GACT_NOISE_REF ? 1 : G.sgr;
  row_grid((supergroups(N, BITS) + sgr - 1) / sgr, &p.grid, &p.block, G.threads);
  // the reference stream's one Philox block per byte makes the kernel instruction-bound: it wants every wave
  p.lds = noise_mode == GACT_NOISE_REF ? 0u : quantize_lds_cap(sizeof(T), BITS, N);
  const bool small = N < G.small_below;
  switch (noise_mode) {
    case GACT_NOISE_CONST: p.kernel = quantize_kernel_of<T, BITS, GACT_NOISE_CONST, GIVEN>(small); break;
    case GACT_NOISE_INJECT: p.kernel = quantize_kernel_of<T, BITS, GACT_NOISE_INJECT, GIVEN>(small); break;
    case GACT_NOISE_REF: p.kernel = quantize_kernel_of<T, BITS, GACT_NOISE_REF, GIVEN>(small); break;
    case GACT_NOISE_FAST: p.kernel = quantize_kernel_of<T, BITS, GACT_NOISE_FAST, GIVEN>(small); break;
  }
  return p;
}

template <typename T, bool GIVEN>
LaunchPlan plan_quantize_bits(int bits, int64_t N, int noise_mode) {
  switch (bits) {
    case 1: return plan_quantize<T, 1, GIVEN>(N, noise_mode);
    case 2: return plan_quantize<T, 2, GIVEN>(N, noise_mode);
    case 4: return plan_quantize<T, 4, GIVEN>(N, noise_mode);
    case 8: return plan_quantize<T, 8, GIVEN>(N, noise_mode);
  }
  return LaunchPlan();
}

// every quantize kernel takes the same arguments
template <typename T, bool GIVEN>
int dispatch_quantize(int bits, const T* x, int64_t numel, int64_t N, uint8_t* packed, typename Elem<T>::Stat* scale,
                      T* mn, T* mx,
                      int noise_mode, SeedArg seed, const float* noise, hipStream_t stream) {
  const LaunchPlan p = plan_quantize_bits<T, GIVEN>(bits, N, noise_mode);
  if (!p.kernel) return GACT_EINVAL;
  void* args[] = {(void*)&seed, (void*)&x, (void*)&numel, (void*)&N, (void*)&packed, (void*)&scale, (void*)&mn, (void*)&mx, (void*)&noise};
  return hipLaunchKernel(p.kernel, p.grid, p.block, args, p.lds, stream) == hipSuccess ? GACT_OK : GACT_ELAUNCH;
}

template <typename T>
LaunchPlan plan_dequantize(int bits, int64_t N) {
  LaunchPlan p;
  // a unit takes 256 / (16 / sizeof(T)) lanes
  const DqGeom d = dq_geom<T>(bits);
  const bool large = N >= d.large_from;
  const int64_t units_per_block = d.threads / (GROUP / (16 / (int64_t)sizeof(T)));
  const int64_t unit_groups = dq_unit_groups(d, bits, large);
  // the caps are stated for workgroups of 256 threads
  p.lds = N >= d.cap_from ? d.lds_large * (unsigned)d.threads / 256u : 0u;
  p.grid = dim3((unsigned)(((N + unit_groups - 1) / unit_groups + units_per_block - 1) / units_per_block));
  p.block = dim3((unsigned)d.threads);
#define GACT_DQ_KERNEL(B) (large ? (const void*)dequantize_kernel<T, B, true> : (const void*)dequantize_kernel<T, B, false>)
  switch (bits) {
    case 1: p.kernel = GACT_DQ_KERNEL(1); break;
    case 2: p.kernel = GACT_DQ_KERNEL(2); break;
    case 4: p.kernel = GACT_DQ_KERNEL(4); break;
    case 8: p.kernel = GACT_DQ_KERNEL(8); break;
  }
#undef GACT_DQ_KERNEL
  return p;
}

template <typename T>
int dispatch_dequantize(int bits, const uint8_t* packed, const typename Elem<T>::Stat* scale, const T* mn,
                        int64_t numel, int64_t N, T* out,
                        hipStream_t stream) {
  const LaunchPlan p = plan_dequantize<T>(bits, N);
  if (!p.kernel) return GACT_EINVAL;
  void* args[] = {(void*)&packed, (void*)&scale, (void*)&mn, (void*)&numel, (void*)&N, (void*)&out};
  return hipLaunchKernel(p.kernel, p.grid, p.block, args, p.lds, stream) == hipSuccess ? GACT_OK : GACT_ELAUNCH;
}

template <typename T>
void launch_minimax_any(const T* x, int64_t N, int64_t D, T* mn, T* mx, hipStream_t stream) {
  const bool vec = aligned16(x);  // D % 32 == 0 keeps every row 16-byte aligned once the base is
  const int64_t pieces = vec ? D / (16 / (int64_t)sizeof(T)) : D;
  int lpr_log2 = 3;
  while (lpr_log2 < 6 && (2LL << lpr_log2) <= pieces) lpr_log2++;
  const bool several = pieces <= (64LL << 1);  // short rows: 4 rows per lane group
  const int64_t groups = several ? (N + 3) / 4 : N;
  const dim3 grid((unsigned)(((groups << lpr_log2) + 255) / 256)), block(256);
  if (vec && several)
    hipLaunchKernelGGL((minimax_any_kernel<T, true, 4>), grid, block, 0, stream, x, N, D, lpr_log2, mn, mx);
  else if (vec)
    hipLaunchKernelGGL((minimax_any_kernel<T, true, 1>), grid, block, 0, stream, x, N, D, lpr_log2, mn, mx);
  else if (several)
    hipLaunchKernelGGL((minimax_any_kernel<T, false, 4>), grid, block, 0, stream, x, N, D, lpr_log2, mn, mx);
  else
    hipLaunchKernelGGL((minimax_any_kernel<T, false, 1>), grid, block, 0, stream, x, N, D, lpr_log2, mn, mx);
}

// the 8-columns-per-thread kernels take G = 1, D % 8 == 0, 16-byte aligned rows, and a thread count that fits 32 bits
inline bool rows8_ok(int bits, int64_t N, int64_t G, int64_t D, uint32_t* tpr, uint32_t* total) {
  if (G != 1 || D % 8 != 0 || D / 8 > 0x7fffffffLL) return false;
  const int64_t rows = supergroups(N, bits), threads = rows * (D / 8);
  if (threads <= 0 || threads > 0xffffff00LL) return false;
  *tpr = (uint32_t)(D / 8);
  *total = (uint32_t)threads;
  return true;
}

template <typename T>
int pack_any(const T* data, const T* mn, const T* scale, int bits, int64_t N, int64_t G, int64_t D, int noise_mode,
             uint64_t seed, const float* noise, uint8_t* packed, hipStream_t stream) {
  uint32_t tpr = 0, threads = 0;
  const bool rows8 = rows8_ok(bits, N, G, D, &tpr, &threads) && aligned16(data) && aligned16(packed) &&
                     (D * (int64_t)sizeof(T)) % 16 == 0 && (noise_mode != GACT_NOISE_INJECT || aligned16(noise));
  const int64_t total = gact_packed_bytes(bits, N, G, D);
  const dim3 grid((unsigned)(rows8 ? (threads + 255u) / 256u : (total + 255) / 256)), block(256);
#define GACT_LAUNCH_PACK(M)                                                                                          \
  do {                                                                                                               \
    if (rows8)                                                                                                       \
      hipLaunchKernelGGL((pack_rows8_kernel<T, M>), grid, block, 0, stream, data, mn, scale, bits, N, tpr, threads,   \
                         seed, noise, packed);                                                                       \
    else                                                                                                             \
      hipLaunchKernelGGL((pack_any_kernel<T, M>), grid, block, 0, stream, data, mn, scale, bits, N, G, D, seed,       \
                         noise, packed, total);                                                                      \
  } while (0)
  switch (noise_mode) {
    case GACT_NOISE_CONST: GACT_LAUNCH_PACK(GACT_NOISE_CONST); break;
    case GACT_NOISE_INJECT: GACT_LAUNCH_PACK(GACT_NOISE_INJECT); break;
    case GACT_NOISE_REF: GACT_LAUNCH_PACK(GACT_NOISE_REF); break;
    case GACT_NOISE_FAST: GACT_LAUNCH_PACK(GACT_NOISE_FAST); break;
    default: return GACT_EINVAL;
  }
#undef GACT_LAUNCH_PACK
  return launch_status();
}

template <typename T>
int unpack_any(const uint8_t* packed, int bits, const T* scale, const T* mn, int64_t N, int64_t G, int64_t D, T* out,
               hipStream_t stream) {
  uint32_t tpr = 0, threads = 0;
  if (rows8_ok(bits, N, G, D, &tpr, &threads) && aligned16(out) && (reinterpret_cast<uintptr_t>(packed) & 7u) == 0 &&
      (D * (int64_t)sizeof(T)) % 16 == 0) {
    hipLaunchKernelGGL((unpack_rows8_kernel<T>), dim3((threads + 255u) / 256u), dim3(256), 0, stream, packed, bits, scale,
                       mn, N, tpr, threads, out);
  } else {
    const int64_t total = gact_packed_bytes(bits, N, G, D);
    hipLaunchKernelGGL((unpack_any_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, packed, bits,
                       scale, mn, N, G, D, out, total);
  }
  return launch_status();
}

}  // namespace

extern "C" {

const char* gact_strerror(int code) {
  switch (code) {
    case GACT_OK: return "ok";
    case GACT_EINVAL: return "invalid argument";
    case GACT_EALIGN: return "pointer is not 16-byte aligned";
    case GACT_ESHAPE: return "unsupported shape";
    case GACT_ELAUNCH: return "HIP launch failed";
    case GACT_EBUDGET: return "bit budget unreachable: every tensor is already at 1 bit";
    case GACT_ELIMIT: return "beyond the limit of the library's own workspace (262144 blocks of 128 groups)";
  }
  return "unknown error";
}

int gact_abi_version(void) { return GACT_ABI_VERSION; }

int64_t gact_packed_bytes(int bits, int64_t N, int64_t G, int64_t D) {
  if (!valid_bits(bits) || N < 0 || G < 0 || D < 0) return GACT_EINVAL;
  const int wpt = 8 / bits;
  const int64_t n_round = (N + wpt - 1) / wpt * wpt;
  return (int64_t)bits * n_round * G * D / 8;
}

int gact_minimax(const void* data, int dtype, int64_t N, int64_t D, void* mn, void* mx, void* stream) {
  if (dtype != GACT_F32 && dtype != GACT_F16) return GACT_EINVAL;
  if (N < 0 || !(D % 32 == 0 && D > 32)) return GACT_ESHAPE;  // minimax_cuda_kernel.cu:80
  if (N == 0) return GACT_OK;
  if (!data || !mn || !mx) return GACT_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  if (D == GROUP && aligned16(data)) {
    dim3 grid, block;
    row_grid((N + MINIMAX_ROW_GROUPS - 1) / MINIMAX_ROW_GROUPS, &grid, &block, MINIMAX_THREADS);
    if (dtype == GACT_F32)
      hipLaunchKernelGGL((minimax256_kernel<float>), grid, block, 0, s, (const float*)data, N, (float*)mn, (float*)mx);
    else
      hipLaunchKernelGGL((minimax256_kernel<f16>), grid, block, 0, s, (const f16*)data, N, (f16*)mn, (f16*)mx);
  } else {
    if (dtype == GACT_F32)
      launch_minimax_any<float>((const float*)data, N, D, (float*)mn, (float*)mx, s);
    else
      launch_minimax_any<f16>((const f16*)data, N, D, (f16*)mn, (f16*)mx, s);
  }
  return launch_status();
}

int gact_pack(const void* data, const void* mn, const void* mx, int dtype, int bits, int64_t N, int64_t G, int64_t D,
              int noise_mode, uint64_t seed, const float* noise, void* packed, void* scale, void* stream) {
  if (dtype != GACT_F32 && dtype != GACT_F16) return GACT_EINVAL;
  if (!valid_bits(bits)) return GACT_EINVAL;  // quantization_cuda_kernel.cu:86
  if (N < 0 || G < 0 || D < 0) return GACT_EINVAL;
  if (noise_mode < GACT_NOISE_CONST || noise_mode > GACT_NOISE_FAST) return GACT_EINVAL;
  if (N * G * D == 0) return GACT_OK;
  if (!data || !mn || !mx || !packed || !scale) return GACT_EINVAL;
  if (noise_mode == GACT_NOISE_INJECT && !noise) return GACT_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  if (G == 1 && D == GROUP && aligned16(data) && aligned16(packed) && (noise_mode != GACT_NOISE_INJECT || aligned16(noise))) {
    // the fused row kernel with min/max taken from the caller
    if (dtype == GACT_F32)
      return dispatch_quantize<float, true>(bits, (const float*)data, N * GROUP, N, (uint8_t*)packed, (float*)scale,
                                            (float*)const_cast<void*>(mn), (float*)const_cast<void*>(mx), noise_mode, SeedArg{seed, nullptr}, noise, s);
    return dispatch_quantize<f16, true>(bits, (const f16*)data, N * GROUP, N, (uint8_t*)packed, (f16*)scale,
                                        (f16*)const_cast<void*>(mn), (f16*)const_cast<void*>(mx), noise_mode, SeedArg{seed, nullptr}, noise, s);
  }
  const int64_t count = N * G;
  const dim3 sgrid((unsigned)((count + 255) / 256)), sblock(256);
  if (dtype == GACT_F32) {
    hipLaunchKernelGGL((scale_kernel<float>), sgrid, sblock, 0, s, (const float*)mn, (const float*)mx, bits, count, (float*)scale);
    return pack_any<float>((const float*)data, (const float*)mn, (const float*)scale, bits, N, G, D, noise_mode, seed, noise, (uint8_t*)packed, s);
  }
  hipLaunchKernelGGL((scale_kernel<f16>), sgrid, sblock, 0, s, (const f16*)mn, (const f16*)mx, bits, count, (f16*)scale);
  return pack_any<f16>((const f16*)data, (const f16*)mn, (const f16*)scale, bits, N, G, D, noise_mode, seed, noise, (uint8_t*)packed, s);
}

int gact_unpack(const void* packed, int bits, const void* scale, const void* mn, int dtype, int64_t N, int64_t G,
                int64_t D, void* out, void* stream) {
  if (dtype != GACT_F32 && dtype != GACT_F16) return GACT_EINVAL;
  if (!valid_bits(bits)) return GACT_EINVAL;  // quantization_cuda_kernel.cu:191
  if (N < 0 || G < 0 || D < 0) return GACT_EINVAL;
  if (N * G * D == 0) return GACT_OK;
  if (!packed || !scale || !mn || !out) return GACT_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  if (G == 1 && D == GROUP && aligned16(out) && aligned16(packed)) {
    if (dtype == GACT_F32)
      return dispatch_dequantize<float>(bits, (const uint8_t*)packed, (const float*)scale, (const float*)mn, N * GROUP, N, (float*)out, s);
    return dispatch_dequantize<f16>(bits, (const uint8_t*)packed, (const f16*)scale, (const f16*)mn, N * GROUP, N, (f16*)out, s);
  }
  if (dtype == GACT_F32)
    return unpack_any<float>((const uint8_t*)packed, bits, (const float*)scale, (const float*)mn, N, G, D, (float*)out, s);
  return unpack_any<f16>((const uint8_t*)packed, bits, (const f16*)scale, (const f16*)mn, N, G, D, (f16*)out, s);
}

int gact_quantize_seeded(const void* x, int dtype, int64_t numel, int bits, int noise_mode, uint64_t seed,
                         const uint64_t* seed_add, const float* noise, void* packed, void* scale, void* mn, void* mx,
                         void* stream) {
  if (dtype != GACT_F32 && dtype != GACT_F16 && dtype != GACT_BF16) return GACT_EINVAL;
  if (!valid_bits(bits) || numel < 0) return GACT_EINVAL;
  if (noise_mode < GACT_NOISE_CONST || noise_mode > GACT_NOISE_FAST) return GACT_EINVAL;
  if (numel == 0) return GACT_OK;
  if (!x || !packed || !scale || !mn) return GACT_EINVAL;
  if (noise_mode == GACT_NOISE_INJECT && !noise) return GACT_EINVAL;
  if (!aligned16(x) || !aligned16(packed) || (noise_mode == GACT_NOISE_INJECT && !aligned16(noise))) return GACT_EALIGN;
  if (reinterpret_cast<uintptr_t>(seed_add) & 7u) return GACT_EALIGN;
  const int64_t N = (numel + GROUP - 1) / GROUP;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  const SeedArg sa{seed, seed_add};
  if (dtype == GACT_F32)
    return dispatch_quantize<float, false>(bits, (const float*)x, numel, N, (uint8_t*)packed, (float*)scale, (float*)mn, (float*)mx, noise_mode, sa, noise, s);
  if (dtype == GACT_BF16)
    return dispatch_quantize<bf16, false>(bits, (const bf16*)x, numel, N, (uint8_t*)packed, (float*)scale, (bf16*)mn, (bf16*)mx, noise_mode, sa, noise, s);
  return dispatch_quantize<f16, false>(bits, (const f16*)x, numel, N, (uint8_t*)packed, (f16*)scale, (f16*)mn, (f16*)mx, noise_mode, sa, noise, s);
}

int gact_quantize(const void* x, int dtype, int64_t numel, int bits, int noise_mode, uint64_t seed, const float* noise,
                  void* packed, void* scale, void* mn, void* mx, void* stream) {
  return gact_quantize_seeded(x, dtype, numel, bits, noise_mode, seed, nullptr, noise, packed, scale, mn, mx, stream);
}

int gact_dequantize(const void* packed, int bits, const void* scale, const void* mn, int dtype, int64_t numel, void* out,
                    void* stream) {
  if (dtype != GACT_F32 && dtype != GACT_F16 && dtype != GACT_BF16) return GACT_EINVAL;
  if (!valid_bits(bits) || numel < 0) return GACT_EINVAL;
  if (numel == 0) return GACT_OK;
  if (!packed || !scale || !mn || !out) return GACT_EINVAL;
  if (!aligned16(out) || !aligned16(packed)) return GACT_EALIGN;
  const int64_t N = (numel + GROUP - 1) / GROUP;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  if (dtype == GACT_F32)
    return dispatch_dequantize<float>(bits, (const uint8_t*)packed, (const float*)scale, (const float*)mn, numel, N, (float*)out, s);
  if (dtype == GACT_BF16)
    return dispatch_dequantize<bf16>(bits, (const uint8_t*)packed, (const float*)scale, (const bf16*)mn, numel, N, (bf16*)out, s);
  return dispatch_dequantize<f16>(bits, (const uint8_t*)packed, (const f16*)scale, (const f16*)mn, numel, N, (f16*)out, s);
}

int gact_launch_geometry(int kind, int dtype, int bits, int64_t N, int* threads, int* lds_bytes, int* workgroups_per_cu) {
  if (dtype != GACT_F32 && dtype != GACT_F16 && dtype != GACT_BF16) return GACT_EINVAL;
  if (!valid_bits(bits) || N <= 0 || (kind != 0 && kind != 1)) return GACT_EINVAL;
  LaunchPlan p;
  if (kind == 0)
    p = dtype == GACT_F32 ? plan_quantize_bits<float, false>(bits, N, GACT_NOISE_FAST)
        : dtype == GACT_F16 ? plan_quantize_bits<f16, false>(bits, N, GACT_NOISE_FAST)
                            : plan_quantize_bits<bf16, false>(bits, N, GACT_NOISE_FAST);
  else
    p = dtype == GACT_F32 ? plan_dequantize<float>(bits, N)
        : dtype == GACT_F16 ? plan_dequantize<f16>(bits, N) : plan_dequantize<bf16>(bits, N);
  if (!p.kernel) return GACT_EINVAL;
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, p.kernel, (int)p.block.x, (size_t)p.lds) != hipSuccess) {
    (void)hipGetLastError();
    return GACT_ELAUNCH;
  }
  if (threads) *threads = (int)p.block.x;
  if (lds_bytes) *lds_bytes = (int)p.lds;
  if (workgroups_per_cu) *workgroups_per_cu = per_cu;
  return GACT_OK;
}

int gact_mask_pack(const uint8_t* data, int64_t n, int32_t* mask, void* stream) {
  if (n < 0) return GACT_EINVAL;
  if (n == 0) return GACT_OK;
  if (!data || !mask) return GACT_EINVAL;
  if (!aligned16(data)) return GACT_EALIGN;
  fresh_launch();
  const int64_t pairs = (n / 512 + 1) / 2;  // pairs of full blocks
  const int64_t waves = (pairs + MASK_PAIRS - 1) / MASK_PAIRS + 1;  // plus the wave that takes the partial block
  hipLaunchKernelGGL(mask_pack_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, (hipStream_t)stream, data, n, mask);
  return launch_status();
}

int gact_mask_unpack(const int32_t* mask, int64_t n, uint8_t* out, void* stream) {
  if (n < 0) return GACT_EINVAL;
  if (n == 0) return GACT_OK;
  if (!mask || !out) return GACT_EINVAL;
  if (!aligned16(out)) return GACT_EALIGN;
  fresh_launch();
  const int64_t blocks = n / 512 + 1;  // the partial block included
  const int64_t waves = (blocks + MASK_STEPS * 4 - 1) / (MASK_STEPS * 4);
  hipLaunchKernelGGL(mask_unpack_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, (hipStream_t)stream, mask, n, out);
  return launch_status();
}

int gact_calc_precision(int32_t* b, const float* C, const int64_t* w, int64_t L, double target) {
  if (L < 0) return GACT_EINVAL;
  if (L == 0) return GACT_OK;
  if (!b || !C || !w) return GACT_EINVAL;
  for (int64_t i = 0; i < L; i++)
    if (!prec_valid_bits(b[i])) return GACT_EINVAL;
  std::priority_queue<std::pair<float, int64_t>> q;
  double b_sum = 0;
  for (int64_t i = 0; i < L; i++)
    if (b[i] > 1) {
      q.push(std::make_pair(prec_key(C[i], b[i], w[i]), i));
      b_sum += (double)((int64_t)b[i] * w[i]);
    }
  while (b_sum > target) {
    if (q.empty()) return GACT_EBUDGET;
    const int64_t i = q.top().second;
    q.pop();
    const int nb = prec_next_bits(b[i]);
    b_sum -= (double)(w[i] * (int64_t)(b[i] - nb));
    b[i] = nb;
    if (nb > 1) q.push(std::make_pair(prec_key(C[i], nb, w[i]), i));
  }
  return GACT_OK;
}

int gact_calc_precision_device(int32_t* b, const float* C, const int64_t* w, int64_t L, double target, int32_t* status,
                               void* stream) {
  if (L < 0) return GACT_EINVAL;
  if (L > PREC_MAX_L) return GACT_ESHAPE;
  if (L == 0) return GACT_OK;
  if (!b || !C || !w) return GACT_EINVAL;
  fresh_launch();
  int64_t M = 4;
  while (M < 4 * L) M <<= 1;
  const size_t lds = (size_t)M * sizeof(uint64_t);
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute((const void*)calc_precision_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
          hipSuccess)
    return GACT_ELAUNCH;
  // one thread per candidate slot up to the largest workgroup: the sort's passes are what the kernel spends its time
  // on (120 tensors: 65.7 us with 64 threads, 25.5 with 256, 22.6 with 512; 24 tensors: 12.0 with 128, 14.1 with 256)
  const unsigned threads = (unsigned)(M < 64 ? 64 : M > PREC_THREADS ? PREC_THREADS : M);
  hipLaunchKernelGGL(calc_precision_kernel, dim3(1), dim3(threads), lds, (hipStream_t)stream, b, C, w,
                     (int)L, target, status);
  return launch_status();
}

int64_t gact_batch_workspace_bytes(int64_t L, int64_t total_blocks) {
  if (L < 0 || L > (1 << 30) || total_blocks < 0 || total_blocks > 0x1fffffffLL) return GACT_EINVAL;
  return batch_workspace_need(L, total_blocks);
}

namespace {
int batch_plan_on(gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks, int64_t capacity,
                  void* workspace, int64_t* verdict, hipStream_t s) {
  const BatchWorkspace ws = batch_workspace(workspace);
  hipLaunchKernelGGL(batch_plan_kernel, dim3((unsigned)(1 + (total_blocks + 255) / 256)), dim3(256), 0, s, table, bits, (int)L,
                     total_blocks, capacity, ws, verdict);
  return launch_status();
}

int quantize_batched_on(const gact_batch_entry* table, const int32_t* bits, int64_t total_blocks, int noise_mode,
                        int dtypes, void* workspace, void* packed_arena, void* scale_arena, void* min_arena,
                        hipStream_t s) {
  const BatchWorkspace ws = batch_workspace(workspace);
  const dim3 grid((unsigned)total_blocks), block(256);
#define GACT_LAUNCH_QB(T, M)                                                                                  \
  hipLaunchKernelGGL((quantize_batched_kernel<T, M>), grid, block, 0, s, table, bits, ws, (uint8_t*)packed_arena, \
                     (uint8_t*)scale_arena, (uint8_t*)min_arena)
#define GACT_LAUNCH_QB_ALL(M)                                                                                 \
  do {                                                                                                        \
    if (dtypes & GACT_DTYPES_F32) GACT_LAUNCH_QB(float, M);                                                   \
    if (dtypes & GACT_DTYPES_F16) GACT_LAUNCH_QB(f16, M);                                                     \
    if (dtypes & GACT_DTYPES_BF16) GACT_LAUNCH_QB(bf16, M);                                                   \
  } while (0)
  switch (noise_mode) {
    case GACT_NOISE_CONST: GACT_LAUNCH_QB_ALL(GACT_NOISE_CONST); break;
    case GACT_NOISE_REF: GACT_LAUNCH_QB_ALL(GACT_NOISE_REF); break;
    default: GACT_LAUNCH_QB_ALL(GACT_NOISE_FAST); break;
  }
#undef GACT_LAUNCH_QB_ALL
#undef GACT_LAUNCH_QB
  return launch_status();
}

inline int batched_args_ok(int64_t L, int64_t total_blocks) {
  return !(L < 0 || L > (1 << 30) || total_blocks < 0 || total_blocks > 0x1fffffffLL);   // the dequantize grid is 4 * total_blocks
}
}  // namespace

int gact_batch_plan(gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks, int64_t capacity,
                    void* workspace, void* stream) {
  if (!batched_args_ok(L, total_blocks) || capacity < 0) return GACT_EINVAL;
  if (!workspace) return GACT_EINVAL;
  if (!aligned16(workspace)) return GACT_EALIGN;
  if (L > 0 && (!table || !bits)) return GACT_EINVAL;
  fresh_launch();
  return batch_plan_on(table, bits, L, total_blocks, capacity, workspace, nullptr, (hipStream_t)stream);
}

int gact_quantize_batched(const gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                          int noise_mode, int dtypes, const void* workspace, void* packed_arena, void* scale_arena,
                          void* min_arena, void* stream) {
  if (!batched_args_ok(L, total_blocks)) return GACT_EINVAL;
  if (noise_mode != GACT_NOISE_CONST && noise_mode != GACT_NOISE_REF && noise_mode != GACT_NOISE_FAST)
    return GACT_EINVAL;  // injected noise is a single-tensor test mode
  if (dtypes < 0 || dtypes > GACT_DTYPES_ALL) return GACT_EINVAL;
  if (dtypes == 0) dtypes = GACT_DTYPES_ALL;
  if (L == 0 || total_blocks == 0) return GACT_OK;
  if (!table || !bits || !workspace || !packed_arena || !scale_arena || !min_arena) return GACT_EINVAL;
  if (!aligned16(packed_arena) || !aligned16(workspace)) return GACT_EALIGN;
  fresh_launch();
  return quantize_batched_on(table, bits, total_blocks, noise_mode, dtypes, const_cast<void*>(workspace), packed_arena,
                             scale_arena, min_arena, (hipStream_t)stream);
}

int gact_dequantize_batched(const gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                            const void* workspace, const void* packed_arena, const void* scale_arena,
                            const void* min_arena, void* stream) {
  if (!batched_args_ok(L, total_blocks)) return GACT_EINVAL;
  if (L == 0 || total_blocks == 0) return GACT_OK;
  if (!table || !bits || !workspace || !packed_arena || !scale_arena || !min_arena) return GACT_EINVAL;
  if (!aligned16(packed_arena) || !aligned16(workspace)) return GACT_EALIGN;
  fresh_launch();
  const dim3 grid((unsigned)(4 * total_blocks)), block(256);
  hipLaunchKernelGGL(dequantize_batched_kernel, grid, block, 0, (hipStream_t)stream, table, bits,
                     batch_workspace(const_cast<void*>(workspace)), (const uint8_t*)packed_arena,
                     (const uint8_t*)scale_arena, (const uint8_t*)min_arena);
  return launch_status();
}

// ------------------------------------------------------------------------------------------------
// The batched quantize for callers that cannot allocate: plan + quantize with the workspace in a device array
// of the library's own.  Every GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends; the address is looked up once per device (the array's name is only a host-side
// handle) and that pointer is what the kernels get.  Calls on one GPU share the array: they must not overlap.
// Nothing in it has to start at zero - the plan kernel writes every field the work kernels read, the verdict
// (`ok`) included, on every call: a void plan left behind by an earlier call cannot leak into the next one.
// The verdict of a call is also written to the caller's `verdict` words, since the array itself is out of reach.
// ------------------------------------------------------------------------------------------------
#define GACT_STATIC_MAX_BLOCKS 262144
#define GACT_STATIC_WORKSPACE_BYTES (256 + GACT_STATIC_MAX_BLOCKS * 4)
#define GACT_MAX_DEVICES 64
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[GACT_STATIC_WORKSPACE_BYTES];

namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[GACT_MAX_DEVICES];  // device address of `scratch` on each device, once looked up

int static_workspace(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= GACT_MAX_DEVICES) return GACT_ELAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return GACT_ELAUNCH;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return GACT_OK;
}
}  // namespace

int gact_quantize_batched_static(gact_batch_entry* table, const int32_t* bits, int64_t L, int64_t total_blocks,
                                 int64_t capacity, int noise_mode, int dtypes, void* packed_arena, void* scale_arena,
                                 void* min_arena, int64_t* verdict, void* stream) {
  if (!batched_args_ok(L, total_blocks) || capacity < 0) return GACT_EINVAL;
  if (noise_mode != GACT_NOISE_CONST && noise_mode != GACT_NOISE_REF && noise_mode != GACT_NOISE_FAST) return GACT_EINVAL;
  if (dtypes < 0 || dtypes > GACT_DTYPES_ALL) return GACT_EINVAL;
  if (dtypes == 0) dtypes = GACT_DTYPES_ALL;
  if (total_blocks > GACT_STATIC_MAX_BLOCKS) return GACT_ELIMIT;
  if (L == 0 || total_blocks == 0) return GACT_OK;
  if (!table || !bits || !packed_arena || !scale_arena || !min_arena) return GACT_EINVAL;
  if (!aligned16(packed_arena)) return GACT_EALIGN;
  if (reinterpret_cast<uintptr_t>(verdict) & 7u) return GACT_EALIGN;
  void* ws = nullptr;
  const int rc = static_workspace(&ws);
  if (rc != GACT_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  fresh_launch();
  const int planned = batch_plan_on(table, bits, L, total_blocks, capacity, ws, verdict, s);
  if (planned != GACT_OK) return planned;
  return quantize_batched_on(table, bits, total_blocks, noise_mode, dtypes, ws, packed_arena, scale_arena, min_arena, s);
}

}  // extern "C"
