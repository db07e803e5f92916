// TEST INFRASTRUCTURE -- not part of the product (see prelude.h).
//
// Key/value radix sort as TensorFrost's own `tf.sort.radix` runs on the C++/OpenMP backend. Follows
// Python/TensorFrost/sort.py:38-187 step by step (CPU branch of the scatter kernel, :122-132):
//   iters = ceil(32/6) = 6 passes of 6 bits, group_size 128, histogram_size 64          (:89-91)
//   per pass: digit = (key >> 6*pass) & 63                                              (:93-94,105)
//     packed group histogram: 4 digits x 8-bit counters per uint, summed over the group (:108-112)
//     unpack to [groups, 64]                                                            (:114-115)
//     inclusive prefix over groups per digit, done in chunks of 64 groups               (:117, :39-50)
//     inclusive prefix over digits of the last row (digit totals)                       (:118-119)
//     scatter: offset = scan[g-1, digit] + total[digit-1] + #{j < e : digit(g, j) == digit}  (:123-132)
//   passes ping-pong keys<->keys1, values<->values1 (two per host-loop iteration)       (:102,173-174)
//   float / int keys go through an order-preserving map to uint and back                (:52-72,82-87,178-182)
// Each step is one generated kernel (one thread per output element, groups spread by OpenMP); the
// loops below keep that thread structure: `omp parallel for` over thread groups, serial inside.
//
// Pins (tests/test_oracle_sort.py): keys and payload against np.argsort(kind="stable") (the reference's
// own test, tests/sorting_test.py:44-54, checks keys against np.argsort); the float map against
// monotonicity on random and special values (+-0, +-inf, denormals, extremes); duplicates-heavy inputs
// so that an unstable scatter fails.

#include <vector>

#include "prelude.h"

using namespace tfo;

namespace {

constexpr int kBits = 6;
constexpr int kHist = 64;
constexpr int kGroup = 128;
constexpr uint kSignBit = 0x80000000u;

inline uint get_bits(uint a, int pass) { return (a >> (pass * kBits)) & (uint)(kHist - 1); }

inline uint map_float_to_uint(uint ux) { return ux ^ (((ux >> 31) == 1u) ? ~0u : kSignBit); }
inline uint map_uint_to_float(uint x) { return x ^ (((x >> 31) == 0u) ? ~0u : kSignBit); }

// [G, 16] packed histogram: thread (g, i) loops over the 128 elements of group g.
void k_group_histogram_packed(const uint* keys, int n, int G, int pass, uint* packed) {
#pragma omp parallel for
	for (int block_id = 0; block_id < (G + 15) / 16; block_id++)
		for (int t1 = 0; t1 < 16; t1++)
			for (int t0 = 0; t0 < 16; t0++) {
				int g = block_id * 16 + t1, i = t0;
				if (g >= G) continue;
				uint sum = 0u;
				for (int e = 0; e < kGroup; e++) {
					int element = g * kGroup + e;
					uint this_key = element < n ? get_bits(keys[element], pass) : 0u;  // split pads with 0
					uint bits = (uint)(this_key == (uint)(4 * i)) + ((uint)(this_key == (uint)(4 * i + 1)) << 8) +
					            ((uint)(this_key == (uint)(4 * i + 2)) << 16) + ((uint)(this_key == (uint)(4 * i + 3)) << 24);
					sum = sum + (element < n ? bits : 0u);
				}
				packed[g * 16 + i] = sum;
			}
}

// [G, 64]: unpack the 8-bit counters.
void k_unpack(const uint* packed, int G, uint* hist) {
#pragma omp parallel for
	for (int g = 0; g < G; g++)
		for (int i = 0; i < kHist; i++) hist[g * kHist + i] = (packed[g * 16 + i / 4] >> (8 * (i % 4))) & 0xFFu;
}

// Inclusive prefix over axis 0 of [G, 64], in chunks of 64 rows: chunk sums, serial scan over chunks,
// then a serial scan inside every chunk seeded with the previous chunk's running total.
void k_prefix_sum_grouped(const uint* hist, int G, uint* scan, std::vector<uint>& chunk_scan) {
	const int chunks = (G + 63) / 64;
	chunk_scan.assign((size_t)chunks * kHist, 0u);
#pragma omp parallel for
	for (int c = 0; c < chunks; c++)
		for (int i = 0; i < kHist; i++) {
			uint sum = 0u;
			for (int e = 0; e < 64; e++) {
				int g = c * 64 + e;
				sum = sum + (g < G ? hist[g * kHist + i] : 0u);
			}
			chunk_scan[(size_t)c * kHist + i] = sum;
		}
	for (int i = 0; i < kHist; i++) {  // one thread per digit, serial over chunks
		uint acc = 0u;
		for (int c = 0; c < chunks; c++) {
			acc = acc + chunk_scan[(size_t)c * kHist + i];
			chunk_scan[(size_t)c * kHist + i] = acc;
		}
	}
#pragma omp parallel for
	for (int c = 0; c < chunks; c++)
		for (int i = 0; i < kHist; i++) {
			uint acc = 0u;
			for (int e = 0; e < 64; e++) {
				int g = c * 64 + e;
				if (g >= G) break;  // merge_dim drops the padded tail
				uint seed = (c == 0 || e != 0) ? 0u : chunk_scan[(size_t)(c - 1) * kHist + i];
				acc = acc + hist[g * kHist + i] + seed;
				scan[g * kHist + i] = acc;
			}
		}
}

// The scatter kernel, CPU branch: kernel shape [G, 128], group {128}.
void k_scatter(const uint* keys_in, const uint* vals_in, uint* keys_out, uint* vals_out, int n, int G, int pass,
               const uint* group_histogram_scan, const uint* total_bit_histogram) {
#pragma omp parallel for
	for (int block_id = 0; block_id < G; block_id++) {
		for (int block_thread_id0 = 0; block_thread_id0 < kGroup; block_thread_id0++) {
			int g = block_id, e = block_thread_id0;
			int element = g * kGroup + e;
			if (element < n) {
				uint old_key = keys_in[element];
				uint bit = get_bits(old_key, pass);
				uint total_offset = (g == 0 ? 0u : group_histogram_scan[(g - 1) * kHist + (int)bit]) +
				                    (bit == 0u ? 0u : total_bit_histogram[bit - 1u]);
				for (int j = 0; j < e; j++) {
					int other = g * kGroup + j;
					uint grouped = other < n ? get_bits(keys_in[other], pass) : 0u;
					total_offset += (uint)(grouped == bit);
				}
				keys_out[total_offset] = old_key;
				if (vals_in) vals_out[total_offset] = vals_in[element];
			}
		}
	}
}

void sort_iteration(const uint* keys_in, uint* keys_out, const uint* vals_in, uint* vals_out, int n, int pass,
                    std::vector<uint>& packed, std::vector<uint>& hist, std::vector<uint>& scan, std::vector<uint>& chunk_scan) {
	const int G = (n + kGroup - 1) / kGroup;
	k_group_histogram_packed(keys_in, n, G, pass, packed.data());
	k_unpack(packed.data(), G, hist.data());
	k_prefix_sum_grouped(hist.data(), G, scan.data(), chunk_scan);
	uint total[kHist];
	uint acc = 0u;
	for (int i = 0; i < kHist; i++) {
		acc = acc + scan[(size_t)(G - 1) * kHist + i];
		total[i] = acc;
	}
	k_scatter(keys_in, vals_in, keys_out, vals_out, n, G, pass, scan.data(), total);
}

}  // namespace

extern "C" {

// key_kind: 0 = uint32, 1 = int32, 2 = float32 (bit patterns passed as uint32). vals_* may be null.
// keys_out / vals_out receive the sorted result; keys_tmp / vals_tmp are n-word work buffers.
int oracle_radix_sort_kv(int key_kind, const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                         uint32_t* keys_tmp, uint32_t* vals_tmp, int n) {
	if (n <= 0) return 0;
	const int G = (n + kGroup - 1) / kGroup;
	std::vector<uint> packed((size_t)G * 16), hist((size_t)G * kHist), scan((size_t)G * kHist), chunk_scan;
	// keys = copy(keys), mapped to uint
#pragma omp parallel for
	for (int i = 0; i < n; i++) {
		uint k = keys_in[i];
		if (key_kind == 2) k = map_float_to_uint(k);
		if (key_kind == 1) k = k ^ kSignBit;
		keys_out[i] = k;
		if (vals_in) vals_out[i] = vals_in[i];
	}
	const int iters = (32 + kBits - 1) / kBits;  // 6
	for (int iter = 0; iter < iters / 2; iter++) {
		sort_iteration(keys_out, keys_tmp, vals_in ? vals_out : nullptr, vals_tmp, n, 2 * iter, packed, hist, scan, chunk_scan);
		sort_iteration(keys_tmp, keys_out, vals_in ? vals_tmp : nullptr, vals_out, n, 2 * iter + 1, packed, hist, scan, chunk_scan);
	}
#pragma omp parallel for
	for (int i = 0; i < n; i++) {
		uint k = keys_out[i];
		if (key_kind == 2) k = map_uint_to_float(k);
		if (key_kind == 1) k = k ^ kSignBit;
		keys_out[i] = k;
	}
	return 0;
}

uint32_t oracle_map_float_to_uint(uint32_t bits) { return map_float_to_uint(bits); }
uint32_t oracle_map_uint_to_float(uint32_t bits) { return map_uint_to_float(bits); }

}  // extern "C"
