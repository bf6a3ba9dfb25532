// Device-side building blocks for the fused blockwise-FP8 quantisation kernels
// (gfx950 / CDNA4, wave64).  No MFMA here: the kernels built on this header are
// HBM-bound; the one contraction of the path has its own file (fq_router.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fq {

// Work-item and workgroup numbers straight from the hardware registers and the kernel's hidden
// arguments.  HIP's threadIdx / blockIdx / gridDim go through device-library functions, and this
// build cannot inline those (the library is compiled with the packed-fp32 feature that the build
// switches off, and a function is not inlined into a caller that lacks one of its target
// features): every use was a real call, with the calling convention's constraints on the
// registers live around it.
__device__ __forceinline__ unsigned tid_x() { return __builtin_amdgcn_workitem_id_x(); }
__device__ __forceinline__ unsigned wg_x() { return __builtin_amdgcn_workgroup_id_x(); }
// The same, opaque to the compiler, for the 128x128 tile code.  From the plain form the compiler
// derives every lane offset and mask of a tile kernel early and keeps them alive (and moves them
// out of any loop over tiles, some thirty registers); with this one each use site starts from
// its own copy of the register and the derived values die where they are used: 4-9 registers
// fewer in every tile kernel (SwiGLU forward 56-61 -> 51-56, RMSNorm tile kernel 58-62 -> 52),
// 1-5 % less time in the SwiGLU and RMSNorm tile kernels.
__device__ __forceinline__ unsigned tile_tid() {
  unsigned t = tid_x();
  asm volatile("" : "+v"(t));
  return t;
}
// number of workgroups of the launch: the first hidden kernel argument (code object v5 and later)
__device__ __forceinline__ unsigned n_wg_x() {
  return ((const __attribute__((address_space(4))) uint32_t*)__builtin_amdgcn_implicitarg_ptr())[0];
}

constexpr int kGroup = 128;           // 1x128 / 128x1 quantisation group
constexpr float kScaleFloor = 1e-30f;  // linghe/tools/util.py:58-60

// FP8 flavours. E4M3 = OCP e4m3fn (max 448), E5M2 = OCP e5m2 (max 57344).
// kE5M2Max448 = e5m2 codes with the scale still derived from 448, which is what
// the reference's group quantiser does when asked for e5m2
// (linghe/quant/group.py:27 divides by 448.0 whatever the output dtype).
enum Fp8Kind : int { kE4M3 = 0, kE5M2 = 1, kE5M2Max448 = 2 };
template <int KIND> struct Fp8Traits;
template <> struct Fp8Traits<kE4M3> { static constexpr float kMax = 448.0f; static constexpr bool kBf8 = false; };
template <> struct Fp8Traits<kE5M2> { static constexpr float kMax = 57344.0f; static constexpr bool kBf8 = true; };
template <> struct Fp8Traits<kE5M2Max448> { static constexpr float kMax = 448.0f; static constexpr bool kBf8 = true; };

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Bulk 16-/8-byte accesses with a choice of cache policy.  STREAM adds the
// non-temporal hint: the line is not kept in L2 or the memory-side cache beyond this
// access.  For data read once or written once it keeps the caches for what IS reused
// (the second read of x after a statistic pass, gathered rows, weights); whether it
// pays is measured per kernel, results are the same either way.
// Every pointer these helpers see is device memory: the explicit global address
// space keeps the accesses global_load/global_store when the pointer was rebuilt from
// scalar registers (a generic pointer would make them flat accesses).
#define FQ_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <bool STREAM>
__device__ __forceinline__ uint4 load16(const void* p) {
  const FQ_GLOBAL u32x4_t* g = (const FQ_GLOBAL u32x4_t*)p;
  u32x4_t t;
  if constexpr (STREAM) t = __builtin_nontemporal_load(g);
  else t = *g;
  return make_uint4(t.x, t.y, t.z, t.w);
}
template <bool STREAM>
__device__ __forceinline__ void store16(void* p, const uint4& v) {
  FQ_GLOBAL u32x4_t* g = (FQ_GLOBAL u32x4_t*)p;
  const u32x4_t t = {v.x, v.y, v.z, v.w};
  if constexpr (STREAM) __builtin_nontemporal_store(t, g);
  else *g = t;
}
template <bool STREAM>
__device__ __forceinline__ void store8(void* p, const uint2& v) {
  FQ_GLOBAL u32x2_t* g = (FQ_GLOBAL u32x2_t*)p;
  const u32x2_t t = {v.x, v.y};
  if constexpr (STREAM) __builtin_nontemporal_store(t, g);
  else *g = t;
}
__device__ __forceinline__ void store_f32(float* p, float v) { *(FQ_GLOBAL float*)p = v; }

// a value every lane of the workgroup holds identically, moved to scalar registers
// so that addresses built from it use a scalar base and 32-bit lane offsets
__device__ __forceinline__ int uniform32(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform64(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// two bf16 packed in a dword -> fp32 (exact)
__device__ __forceinline__ float bf16_lo(uint32_t p) { return as_f32(p << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t p) { return as_f32(p & 0xffff0000u); }

// 8 packed bf16 (one 128-bit load) -> 8 fp32
__device__ __forceinline__ void unpack8(const uint4& p, float (&v)[8]) {
  v[0] = bf16_lo(p.x); v[1] = bf16_hi(p.x);
  v[2] = bf16_lo(p.y); v[3] = bf16_hi(p.y);
  v[4] = bf16_lo(p.z); v[5] = bf16_hi(p.z);
  v[6] = bf16_lo(p.w); v[7] = bf16_hi(p.w);
}

// per-row weight of the weighted SwiGLU forms: [M] fp32 or bf16, nullptr = unweighted
struct RowWeight {
  const void* w;
  int is_bf16;
};
// R weights of rows r[0..R-1] (all of them valid addresses) as loaded, to be widened where they are
// used (weight_from_bits): no arithmetic on them here, hence no wait, and one branch on the weight's
// type around R straight loads, so that they are in flight together
template <int R>
__device__ __forceinline__ void load_weight_bits(const RowWeight& w, const int64_t (&r)[R], uint32_t (&bits)[R]) {
  if (w.is_bf16) {
#pragma unroll
    for (int s = 0; s < R; ++s) bits[s] = (uint32_t)((const uint16_t*)w.w)[r[s]];
  } else {
#pragma unroll
    for (int s = 0; s < R; ++s) bits[s] = ((const uint32_t*)w.w)[r[s]];
  }
}
// The weight of a row that is the same in every lane of the wave (wave-per-row kernels): a scalar
// load through the constant path, which neither queues behind the wave's vector loads nor counts
// against their wait counter.  A bf16 weight is read as the aligned 4-byte word that holds it (the
// word may reach two bytes beyond either end of the array, never beyond the word of a valid element).
__device__ __forceinline__ float load_weight_uniform(const RowWeight& w, int64_t r) {
  typedef const __attribute__((address_space(4))) uint32_t* const_u32;
  if (w.is_bf16) {
    const uintptr_t at = (uintptr_t)w.w + 2 * (uintptr_t)r;  // the array may start on an odd element of its storage
    const uint32_t d = *(const_u32)(at & ~(uintptr_t)3);
    return as_f32((at & 2) ? (d & 0xffff0000u) : (d << 16));
  }
  return as_f32(((const_u32)(uintptr_t)w.w)[r]);
}
__device__ __forceinline__ float weight_from_bits(const RowWeight& w, uint32_t bits) {
  return as_f32(bits << (w.is_bf16 ? 16 : 0));
}

// fp32 pair -> packed bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  floatx2_t f = {a, b};
  bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint4 pack8_bf16(const float (&v)[8]) {
  uint4 o;
  o.x = pack_bf16x2(v[0], v[1]);
  o.y = pack_bf16x2(v[2], v[3]);
  o.z = pack_bf16x2(v[4], v[5]);
  o.w = pack_bf16x2(v[6], v[7]);
  return o;
}

// sum of squares of 8 packed bf16 with the bf16 dot-product instruction: the
// products are exact in fp32, the additions round in a fixed order
__device__ __forceinline__ float sumsq8(const uint4& p) {
  float ss = 0.f;
  ss = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p.x), __builtin_bit_cast(bf16x2_t, p.x), ss, false);
  ss = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p.y), __builtin_bit_cast(bf16x2_t, p.y), ss, false);
  ss = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p.z), __builtin_bit_cast(bf16x2_t, p.z), ss, false);
  ss = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p.w), __builtin_bit_cast(bf16x2_t, p.w), ss, false);
  return ss;
}

// 4 fp32 -> 4 fp8 codes in one dword (native converts, RNE)
template <int KIND>
__device__ __forceinline__ uint32_t pack4_fp8(float a, float b, float c, float d) {
  // both halves of w are written by the two converts; seeding it with a's bits (a is
  // dead after this) lets the first convert work in place instead of clearing a register
  uint32_t w = as_u32(a);
  if constexpr (!Fp8Traits<KIND>::kBf8) {
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  } else {
    w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, w, true);
  }
  return w;
}

typedef short i16x2_t __attribute__((ext_vector_type(2)));
// codes of a/s, b/s, c/s, d/s for a power-of-two s (exact quotients, RNE)
template <int KIND>
__device__ __forceinline__ uint32_t pack4_fp8_scaled(float a, float b, float c, float d, float s) {
  i16x2_t w = __builtin_bit_cast(i16x2_t, as_u32(a));
  if constexpr (!Fp8Traits<KIND>::kBf8) {
    w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w, a, b, s, false);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w, c, d, s, true);
  } else {
    w = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(w, a, b, s, false);
    w = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(w, c, d, s, true);
  }
  return __builtin_bit_cast(uint32_t, w);
}

// ---------------------------------------------------------------------------
// Division by a scale that is shared by many elements, in two operations each.
//   per scale:   r  = 1/s, v_rcp_f32 plus one Newton step
//                rl = fl((1 - s*r) * r): the part of 1/s that r misses, so that
//                     r + rl = 1/s to about 2^-48 (the residual 1 - s*r is exact in an fma)
//   per element: q  = fma(v, r, fl(v * rl))
// q is the exact v*r plus a correction good to 2^-24 of itself, rounded once: the
// correctly rounded v/s unless v/s lies within ~2^-48 (relative) of the midpoint of two
// floats.  Against IEEE division on the CPU: 4 of 10^9 random quotients differ, by one
// fp32 ulp, and such a difference reaches an FP8 code only if the quotient also sits
// on an FP8 rounding boundary (2^-19 of those): never observed, ~10^-14 per element.
// (The plain product v*r is off by an ulp often enough to flip 3 codes in 10^7.)
// A zero keeps no sign: (-0)/s comes out as +0, whose code differs in the sign bit only.
// ---------------------------------------------------------------------------
struct Divisor {
  float r;   // ~ 1/s
  float rl;  // 1/s - r
};
__device__ __forceinline__ Divisor make_divisor(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  const float r = __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
  Divisor d;
  d.r = r;
  d.rl = __builtin_fmaf(-s, r, 1.0f) * r;
  return d;
}
__device__ __forceinline__ float div_by_scale(float v, const Divisor& d) {
  return __builtin_fmaf(v, d.r, v * d.rl);
}

// What the quantisers keep per scale.  POW2 (round_scale): the scale is a power of two
// and rides in the convert instruction itself (v_cvt_scalef32_pk_*: codes of v / scale,
// only the exponent of the scale operand is used), so there is no arithmetic per
// element at all; otherwise the two terms of the reciprocal.
template <bool POW2>
struct Quantum {
  float a, b;  // POW2: a = scale;  else {a, b} = Divisor{r, rl}
};
template <bool POW2>
__device__ __forceinline__ Quantum<POW2> make_quantum(float s) {
  Quantum<POW2> q;
  if constexpr (POW2) {
    q.a = s;
    q.b = 0.f;
  } else {
    const Divisor d = make_divisor(s);
    q.a = d.r;
    q.b = d.rl;
  }
  return q;
}

// codes of four values under one scale
template <int KIND, bool POW2>
__device__ __forceinline__ uint32_t quantize4(float a, float b, float c, float d, const Quantum<POW2>& q) {
  if constexpr (POW2) {
    return pack4_fp8_scaled<KIND>(a, b, c, d, q.a);
  } else {
    const Divisor dv{q.a, q.b};
    return pack4_fp8<KIND>(div_by_scale(a, dv), div_by_scale(b, dv), div_by_scale(c, dv), div_by_scale(d, dv));
  }
}
template <int KIND, bool POW2>
__device__ __forceinline__ uint2 quantize8(const float (&v)[8], const Quantum<POW2>& q) {
  uint2 pk;
  pk.x = quantize4<KIND, POW2>(v[0], v[1], v[2], v[3], q);
  pk.y = quantize4<KIND, POW2>(v[4], v[5], v[6], v[7], q);
  return pk;
}

// exp2(ceil(log2(s))) as torch evaluates it in fp32 (linghe/tools/util.py:61-62):
// the fp32 log2 of a value a few ulps above 2^e rounds to e itself, so such
// values are NOT rounded up.  Reproduced with integer arithmetic: round up iff
// log2(mantissa) exceeds half an fp32 ulp of the number line just above e.
__device__ __forceinline__ float pow2_ceil_like_torch(float s) {
  uint32_t b = as_u32(s);
  int e = (int)((b >> 23) & 0xffu) - 127;
  uint32_t k = b & 0x7fffffu;
  if (k != 0) {
    bool up = true;
    if (e != 0) {
      uint32_t ae = (uint32_t)(e < 0 ? -e : e);
      int fl = 31 - __builtin_clz(ae);
      bool pow2 = (ae & (ae - 1u)) == 0u;
      int ulp_exp = fl - 23 - ((e < 0 && pow2) ? 1 : 0);
      float half_ulp = as_f32((uint32_t)(ulp_exp - 1 + 127) << 23);
      float delta = (float)k * (1.4426950408889634f * 0x1p-23f);
      up = delta > half_ulp;
    }
    if (up) e += 1;
  }
  return as_f32((uint32_t)(e + 127) << 23);
}

// scale = max(amax / fmax, 1e-30) [rounded up to a power of two]
template <int KIND, bool ROUND>
__device__ __forceinline__ float make_scale(float amax) {
  float s = fmaxf(amax / Fp8Traits<KIND>::kMax, kScaleFloor);
  if constexpr (ROUND) s = pow2_ceil_like_torch(s);
  return s;
}

// ---------------------------------------------------------------------------
// DPP reductions inside a row of 16 lanes (a wave64 is four such rows).
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return as_f32((uint32_t)__builtin_amdgcn_mov_dpp((int)as_u32(v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

// every lane of the 16-lane row ends with the max over the row
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_mov<kDppQuadXor1>(v));
  v = fmaxf(v, dpp_mov<kDppQuadXor2>(v));
  v = fmaxf(v, dpp_mov<kDppRowHalfMirror>(v));
  v = fmaxf(v, dpp_mov<kDppRowMirror>(v));
  return v;
}
// every lane of the 16-lane row ends with the same sum (fixed order -> deterministic)
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_mov<kDppQuadXor1>(v);
  v += dpp_mov<kDppQuadXor2>(v);
  v += dpp_mov<kDppRowHalfMirror>(v);
  v += dpp_mov<kDppRowMirror>(v);
  return v;
}
// whole-wave sum / max, result in every lane
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// the same for a double (two dwords per DPP move): used where a sum has to come
// out independent of the order of its terms
template <int CTRL>
__device__ __forceinline__ double dpp_mov_d(double v) {
  const uint64_t u = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)u, CTRL, 0xf, 0xf, true);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(u >> 32), CTRL, 0xf, 0xf, true);
  return __builtin_bit_cast(double, (uint64_t)lo | ((uint64_t)hi << 32));
}
// every lane of the 16-lane row ends with the same sum
__device__ __forceinline__ double row16_sum_d(double v) {
  v += dpp_mov_d<kDppQuadXor1>(v);
  v += dpp_mov_d<kDppQuadXor2>(v);
  v += dpp_mov_d<kDppRowHalfMirror>(v);
  v += dpp_mov_d<kDppRowMirror>(v);
  return v;
}
__device__ __forceinline__ double wave_sum_d(double v) {
  v = row16_sum_d(v);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// Scheduling fences for the register allocator.  The compiler likes to widen the packed bf16
// rows of a tile as soon as they arrive, long before the arithmetic that uses them; the fp32
// copies (twice the registers) then sit beside the results of earlier rows and push a kernel
// over its register cap.  fence_values / fence_packed cost no instruction: they are empty
// volatile asm statements (which keep their order among themselves) that claim to rewrite
// their operands, so whatever is computed from a fenced packed row starts after the fenced
// results before it are complete.
__device__ __forceinline__ void fence_values(float (&v)[8]) {
  asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
}
__device__ __forceinline__ void fence_packed(uint4& p) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));  // one 128-bit operand: the four dwords stay a tuple
  u32x4 t = __builtin_bit_cast(u32x4, p);
  asm volatile("" : "+v"(t));
  p = __builtin_bit_cast(uint4, t);
}

// sigmoid(x) = 1 / (1 + exp(-x)):
//   exp(-x) = exp2(-x*log2(e)) with v_exp_f32 (1 ulp). A single fp32 product
//   x * -log2(e) would round the exponent and cost up to |x|*4e-8 of relative error
//   (11 ulp of the sigmoid at x = -8), so -log2(e) is split into a 16-bit head,
//   whose product with a bf16-valued x (8 significant bits) is exact, and a tail
//   applied to first order: exp2(hi + lo) = exp2(hi) * (1 + lo*ln2), |lo*ln2| < 1e-3.
//   For an x with more than 8 significant bits the head product rounds and the old
//   bound applies; every caller passes widened bf16 data.
//   The reciprocal is v_rcp_f32 plus one Newton step (correctly rounded but for
//   ~1e-6 of the inputs).
// The exponent is clamped so that 1 + exp(-x) stays finite: for x < -87 the result
// is 2^-126 instead of 0, far below anything a code or a scale can see.
__device__ __forceinline__ float sigmoid_f32(float x) {
  constexpr float kHead = -1.44268798828125f;         // -log2(e) to 16 significant bits
  constexpr float kTailLn2 = -4.888495368504664e-06f; // (-log2(e) - kHead) * ln(2)
  const float e0 = __builtin_amdgcn_exp2f(fminf(x * kHead, 126.0f));
  const float d = 1.0f + __builtin_fmaf(e0, x * kTailLn2, e0);
  const float r0 = __builtin_amdgcn_rcpf(d);
  const float err = __builtin_fmaf(-d, r0, 1.0f);
  return __builtin_fmaf(err, r0, r0);
}

}  // namespace fq
