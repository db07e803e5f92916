#include "hip_generator.h"

#include <cmath>
#include <cstdio>
#include <set>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

namespace tfhost {

static const char* TypeName(TFType t) {
	switch (t) {
		case TFType_Float: return "float";
		case TFType_Uint: return "uint";
		case TFType_Int: return "int";
		case TFType_Bool: return "bool";
		default: return "void";
	}
}

std::string FormatFloat(double value) {
	float f = (float)value;
	if (!std::isfinite(f)) {
		char buf[48];
		snprintf(buf, sizeof(buf), "__uint_as_float(0x%08xu)", FloatBits(f));
		return buf;
	}
	// Nine significant digits reproduce any float exactly.
	char buf[48];
	snprintf(buf, sizeof(buf), "%.9g", (double)f);
	std::string s(buf);
	if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
	if (s.find('.') == std::string::npos) {  // "1e+10" -> "1.0e+10"
		size_t e = s.find('e');
		s = s.substr(0, e) + ".0" + s.substr(e);
	}
	return s + "f";
}

std::string GetHIPHeader() {
	return R"(typedef unsigned int uint;

// ---- helpers of generated kernels (semantics of the C++/OpenMP backend's prelude) ----
__device__ __forceinline__ int tf_min(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int tf_max(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ uint tf_min(uint a, uint b) { return a < b ? a : b; }
__device__ __forceinline__ uint tf_max(uint a, uint b) { return a > b ? a : b; }
__device__ __forceinline__ float tf_min(float a, float b) { return a < b ? a : b; }
__device__ __forceinline__ float tf_max(float a, float b) { return a > b ? a : b; }
__device__ __forceinline__ float asfloat(uint x) { return __uint_as_float(x); }
__device__ __forceinline__ float asfloat(int x) { return __int_as_float(x); }
__device__ __forceinline__ float asfloat(float x) { return x; }
__device__ __forceinline__ uint asuint(float x) { return __float_as_uint(x); }
__device__ __forceinline__ uint asuint(int x) { return (uint)x; }
__device__ __forceinline__ uint asuint(uint x) { return x; }
__device__ __forceinline__ uint asuint(bool x) { return x ? 1u : 0u; }
__device__ __forceinline__ int asint(uint x) { return (int)x; }
__device__ __forceinline__ int asint(float x) { return __float_as_int(x); }
__device__ __forceinline__ int asint(int x) { return x; }
__device__ __forceinline__ int asint(bool x) { return x ? 1 : 0; }
__device__ __forceinline__ bool asbool(uint x) { return x != 0u; }
__device__ __forceinline__ bool asbool(int x) { return x != 0; }
__device__ __forceinline__ bool asbool(bool x) { return x; }
__device__ __forceinline__ int tf_clamp(int x, int a, int b) { return tf_min(tf_max(x, a), b); }
__device__ __forceinline__ uint tf_clamp(uint x, uint a, uint b) { return tf_min(tf_max(x, a), b); }
__device__ __forceinline__ float tf_clamp(float x, float a, float b) { return tf_min(tf_max(x, a), b); }
// A word that this kernel reads once (the operand of a reduction loop): not kept in the caches.
__device__ __forceinline__ uint tf_stream_load(const uint* p) { return __builtin_nontemporal_load(p); }
// An index clamp inside a loop that is emitted in two forms: the form entered after a run-time test that the clamp
// changes nothing redefines this as the identity.
#define TF_INDEX_CLAMP(x, lo, hi) tf_clamp(x, lo, hi)
__device__ __forceinline__ float tf_lerp(float a, float b, float t) { return a + (b - a) * t; }
__device__ __forceinline__ float tf_smoothstep(float a, float b, float t) {
  t = tf_clamp((t - a) / (b - a), 0.0f, 1.0f);
  return t * t * (3.0f - 2.0f * t);
}
__device__ __forceinline__ float tf_sign(float x) { return x < 0.0f ? -1.0f : 1.0f; }
__device__ __forceinline__ int tf_sign(int x) { return x < 0 ? -1 : 1; }
__device__ __forceinline__ float tf_abs(float x) { return fabsf(x); }
__device__ __forceinline__ int tf_abs(int x) { return x < 0 ? -x : x; }
__device__ __forceinline__ uint tf_abs(uint x) { return x; }
__device__ __forceinline__ uint reversebits(uint x) { return __brev(x); }
__device__ __forceinline__ int reversebits(int x) { return (int)__brev((uint)x); }
__device__ __forceinline__ uint pcg(uint v) {
  uint state = v * 747796405u + 2891336453u;
  uint word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
  return (word >> 22u) ^ word;
}
__device__ __forceinline__ float pcgf(uint v) { return (float)pcg(v) / (float)0xffffffffu; }
// Operations the C++ prelude does not define (those programs cannot run on the CPU backend).
// Division, reciprocal and square roots. The reference compiles its kernels with -ffast-math
// (Backend.cpp:35), which licenses reciprocal-based division; here they are the single hardware
// instructions (1 ulp each, quotient within 2 ulp; operands below 2^-126 or quotients of divisors
// above 2^126 lose their denormal range). -DTF_PRECISE_MATH in the backend options selects the
// correctly rounded sequences (about 12 more instructions per division, 20 per square root).
#ifdef TF_PRECISE_MATH
#define TF_REASSOC(reordered, written) (written)
__device__ __forceinline__ float tf_div(float a, float b) { return a / b; }
__device__ __forceinline__ float tf_div_by_pow_3_2(float a, float y) { return a / (y * sqrtf(y)); }
__device__ __forceinline__ float tf_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ float tf_rsqrt(float x) { return rsqrtf(x); }
__device__ __forceinline__ float tf_rcp(float x) { return 1.0f / x; }
#else
#define TF_REASSOC(reordered, written) (reordered)
__device__ __forceinline__ float tf_div(float a, float b) { return a * __builtin_amdgcn_rcpf(b); }
__device__ __forceinline__ float tf_div_by_pow_3_2(float a, float y) {
  const float r = __builtin_amdgcn_rsqf(y);
  return a * (r * r * r);
}
__device__ __forceinline__ float tf_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ float tf_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float tf_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
#endif
__device__ __forceinline__ float tf_frac(float x) { return x - floorf(x); }
__device__ __forceinline__ float tf_step(float edge, float x) { return x >= edge ? 1.0f : 0.0f; }
__device__ __forceinline__ void group_barrier() { __syncthreads(); }
// Integer remainder by a run-time divisor. Same value as C's a % b for every input; operands that are
// already in [0, b) or one period above it (periodic-boundary indices such as (i + N - 1) % N) skip the
// ~30-instruction division sequence.
__device__ __forceinline__ int tf_mod(int a, int b) {
  if (b > 0) {
    if ((uint)a < (uint)b) return a;
    const int d = a - b;
    if ((uint)d < (uint)b) return d;
  }
  return a % b;
}
__device__ __forceinline__ uint tf_mod(uint a, uint b) {
  if (a < b) return a;
  const uint d = a - b;
  if (d < b) return d;
  return a % b;
}

// Four consecutive words at any 4-byte-aligned address as one memory instruction.
typedef uint tf_uint4 __attribute__((ext_vector_type(4)));
typedef tf_uint4 tf_uint4_a4 __attribute__((aligned(4)));
__device__ __forceinline__ tf_uint4 tf_load4(const uint* p) { return *(const tf_uint4_a4*)p; }
__device__ __forceinline__ tf_uint4 tf_load4_stream(const uint* p) { return __builtin_nontemporal_load((const tf_uint4_a4*)p); }
__device__ __forceinline__ void tf_store4(uint* p, uint a, uint b, uint c, uint d) {
  tf_uint4 v = {a, b, c, d};
  *(tf_uint4_a4*)p = v;
}

// ---- atomics on word buffers ----
__device__ __forceinline__ void InterlockedAdd(int* m, int a, int v) { atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedAdd(uint* m, int a, uint v) { atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedAdd(float* m, int a, float v) { atomicAdd(m + a, v); }
__device__ __forceinline__ int InterlockedAdd_Prev(int* m, int a, int v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ uint InterlockedAdd_Prev(uint* m, int a, uint v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ float InterlockedAdd_Prev(float* m, int a, float v) { return atomicAdd(m + a, v); }
__device__ __forceinline__ void InterlockedMin(int* m, int a, int v) { atomicMin(m + a, v); }
__device__ __forceinline__ void InterlockedMin(uint* m, int a, uint v) { atomicMin(m + a, v); }
__device__ __forceinline__ void InterlockedMax(int* m, int a, int v) { atomicMax(m + a, v); }
__device__ __forceinline__ void InterlockedMax(uint* m, int a, uint v) { atomicMax(m + a, v); }
__device__ __forceinline__ void InterlockedMin(float* m, int a, float v) {
  uint* p = (uint*)(m + a);
  uint old = *p;
  while (true) {
    float cur = __uint_as_float(old);
    float goal = tf_min(cur, v);
    if (__float_as_uint(goal) == old) break;
    uint seen = atomicCAS(p, old, __float_as_uint(goal));
    if (seen == old) break;
    old = seen;
  }
}
__device__ __forceinline__ void InterlockedMax(float* m, int a, float v) {
  uint* p = (uint*)(m + a);
  uint old = *p;
  while (true) {
    float cur = __uint_as_float(old);
    float goal = tf_max(cur, v);
    if (__float_as_uint(goal) == old) break;
    uint seen = atomicCAS(p, old, __float_as_uint(goal));
    if (seen == old) break;
    old = seen;
  }
}
__device__ __forceinline__ void InterlockedAnd(int* m, int a, int v) { atomicAnd(m + a, v); }
__device__ __forceinline__ void InterlockedAnd(uint* m, int a, uint v) { atomicAnd(m + a, v); }
__device__ __forceinline__ void InterlockedOr(int* m, int a, int v) { atomicOr(m + a, v); }
__device__ __forceinline__ void InterlockedOr(uint* m, int a, uint v) { atomicOr(m + a, v); }
__device__ __forceinline__ void InterlockedXor(int* m, int a, int v) { atomicXor(m + a, v); }
__device__ __forceinline__ void InterlockedXor(uint* m, int a, uint v) { atomicXor(m + a, v); }

// ---- cross-lane finish of a cooperative reduction: over the whole wave, or over aligned groups of `width` lanes ----
#define TF_WAVE_REDUCE(T, NAME, EXPR)                                  \
  __device__ __forceinline__ T NAME(T a, int width = 64) {             \
    _Pragma("unroll") for (int off = 32; off >= 1; off >>= 1) {        \
      if (off < width) {                                               \
        T b = __shfl_xor(a, off, 64);                                  \
        a = (EXPR);                                                    \
      }                                                                \
    }                                                                  \
    return a;                                                          \
  }
TF_WAVE_REDUCE(float, tf_wave_add, a + b)
TF_WAVE_REDUCE(int, tf_wave_add, a + b)
TF_WAVE_REDUCE(uint, tf_wave_add, a + b)
TF_WAVE_REDUCE(float, tf_wave_mul, a * b)
TF_WAVE_REDUCE(int, tf_wave_mul, a * b)
TF_WAVE_REDUCE(uint, tf_wave_mul, a * b)
TF_WAVE_REDUCE(float, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(int, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(uint, tf_wave_max, tf_max(a, b))
TF_WAVE_REDUCE(float, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(int, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(uint, tf_wave_min, tf_min(a, b))
TF_WAVE_REDUCE(int, tf_wave_and, a & b)
TF_WAVE_REDUCE(uint, tf_wave_and, a & b)
TF_WAVE_REDUCE(int, tf_wave_or, a | b)
TF_WAVE_REDUCE(uint, tf_wave_or, a | b)
__device__ __forceinline__ unsigned long long tf_group_votes(bool a, int width) {
  const unsigned long long votes = __ballot(a);
  if (width == 64) return votes;
  return (votes >> ((threadIdx.x & 63u) & ~(unsigned)(width - 1))) & ((1ull << width) - 1ull);
}
__device__ __forceinline__ bool tf_wave_and(bool a, int width = 64) { return width == 64 ? __all(a) : tf_group_votes(a, width) == (1ull << width) - 1ull; }
__device__ __forceinline__ bool tf_wave_or(bool a, int width = 64) { return width == 64 ? __any(a) : tf_group_votes(a, width) != 0ull; }

)";
}

}  // namespace tfhost
