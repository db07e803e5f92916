// TEST INFRASTRUCTURE -- not part of the product (see prelude.h). C entry points over the prelude helpers so
// that tests can pin them one by one.
#include "prelude.h"

using namespace tfo;

extern "C" {
uint32_t oracle_pcg(uint32_t v) { return pcg(v); }
float oracle_pcgf(uint32_t v) { return pcgf(v); }
uint32_t oracle_reversebits(uint32_t v) { return reversebits(v); }
float oracle_sign_f(float x) { return sign(x); }
int oracle_sign_i(int x) { return sign(x); }
int oracle_clamp_i(int x, int a, int b) { return clamp(x, a, b); }
float oracle_clamp_f(float x, float a, float b) { return clamp(x, a, b); }
float oracle_lerp(float a, float b, float t) { return lerp(a, b, t); }
float oracle_smoothstep(float a, float b, float t) { return smoothstep(a, b, t); }
float oracle_max_f(float a, float b) { return max(a, b); }
float oracle_min_f(float a, float b) { return min(a, b); }
uint32_t oracle_asuint_f(float x) { return asuint(x); }
float oracle_asfloat_u(uint32_t x) { return asfloat(x); }
size_t oracle_work_group_count(const size_t* shape, size_t dispatch_dim, const size_t* group, size_t group_dim) {
	return work_group_count(shape, dispatch_dim, group, group_dim);
}
}
