// Stable least-significant-digit radix sort of 32-bit keys with an optional 32-bit payload.
//
// The reference's sort is a Python composition of ordinary tensor ops (Python/TensorFrost/sort.py:38-187):
// 6 passes of 6 bits, each pass a packed per-group histogram (:105-115), a grouped prefix sum over the
// [groups, 64] histogram matrix (:117, :39-50), digit totals (:118-119) and a scatter kernel that finds
// an element's rank by re-scanning its 128-element group (:121-169) -- about 7 kernels and >= 100 B of
// memory traffic per key per sort, plus float/int keys remapped to order-preserving uints (:52-72).
//
// Here: 8-bit digits, 4 passes, "onesweep":
//   1. one histogram kernel reads the keys once and counts all four digits; a one-group kernel turns the
//      counts into exclusive digit offsets;
//   2. one kernel per pass. A 1024-thread group owns a tile of 16384 keys, ranks them by digit with
//      wave-wide match operations (stable: ties keep memory order), resolves for each of the 256 digits
//      how many keys with that digit precede the tile by looking back over the counts that earlier tiles
//      published (decoupled look-back, tiles ordered by a ticket), sorts the tile by digit through LDS and
//      writes keys and payload to their final places in runs that are contiguous per digit.
// Traffic per key: 4 B (histogram) + 4 x (8 B read + 8 B write) with payload.
//
// Key kinds (as sort.py:52-72): u32 as is; i32 with the sign bit flipped; f32 with all bits flipped for
// negatives and the sign bit flipped otherwise. The mapping is applied when pass 0 loads and undone when
// the last pass stores.

#include "common.h"

namespace tfhip {

constexpr int kRsThreads = 1024;
constexpr int kRsWaves = kRsThreads / 64;
constexpr int kRsItems = 16;
constexpr int kRsTile = kRsThreads * kRsItems;  // 16384
constexpr int kRsWaveSpan = 64 * kRsItems;      // keys one wave owns: 1024 consecutive
constexpr int kRadix = 256;
constexpr uint32_t kRsSpinLimit = 1u << 22;
constexpr int kLookWindow = 8;  // earlier tiles examined per step of the look-back

constexpr uint32_t kStAggregate = 1u << 30;
constexpr uint32_t kStPrefix = 2u << 30;
constexpr uint32_t kStValueMask = (1u << 30) - 1;

enum KeyKind { kKeyU32 = 0, kKeyI32 = 1, kKeyF32 = 2 };

__device__ __forceinline__ uint32_t key_encode(uint32_t k, int kind) {
	if (kind == kKeyI32) return k ^ 0x80000000u;
	if (kind == kKeyF32) return k ^ ((k >> 31) ? 0xFFFFFFFFu : 0x80000000u);
	return k;
}
__device__ __forceinline__ uint32_t key_decode(uint32_t k, int kind) {
	if (kind == kKeyI32) return k ^ 0x80000000u;
	if (kind == kKeyF32) return k ^ ((k >> 31) ? 0x80000000u : 0xFFFFFFFFu);
	return k;
}

__device__ __forceinline__ void st_store(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t st_load(uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// ---- 1. digit histograms ------------------------------------------------------------------------

// hist[pass*256 + digit] += occurrences, all four digits from one read of the keys. Group-stride loop over tiles of
// 8192 keys, four keys per lane and load. Every counter exists kHistCopies times in group memory, the copy chosen by
// the lane, so the 64 adds of a wave spread over the banks whatever the digits are (equal digits included: sorted
// or low-entropy input needs no special case); one counter per digit made the kernel wait on bank conflicts and
// same-address adds (2^28 keys: 560 us, against about 290 us with the copies; fetching the next tile while one is
// counted changes nothing, so what remains is the rate of the adds themselves).
constexpr int kHistCopies = 16;  // 4 digits x 256 bins x 16 copies x 4 B = 64 KiB
constexpr int kHistThreads = 512, kHistItems = 16, kHistTile = kHistThreads * kHistItems;

__device__ __forceinline__ void histogram_add(uint32_t* lds, uint32_t key, int copy) {
#pragma unroll
	for (int p = 0; p < 4; p++) atomicAdd(&lds[((p * kRadix) + ((key >> (8 * p)) & 255u)) * kHistCopies + copy], 1u);
}

__global__ __launch_bounds__(kHistThreads) void radix_histogram_kernel(const uint32_t* __restrict__ keys, size_t n, uint32_t* __restrict__ hist, int kind) {
	__shared__ uint32_t lds[4 * kRadix * kHistCopies];
	for (int i = threadIdx.x; i < 4 * kRadix * kHistCopies; i += kHistThreads) lds[i] = 0;
	__syncthreads();
	const int copy = threadIdx.x & (kHistCopies - 1);
	const size_t tiles = (n + kHistTile - 1) / kHistTile;
	const bool aligned = (reinterpret_cast<uintptr_t>(keys) & 15) == 0;
	for (size_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
		const size_t base = tile * kHistTile;
		if (aligned && base + kHistTile <= n) {
			constexpr int kVecs = kHistTile / (4 * kHistThreads);  // 16-byte loads per lane
			uint4 v[kVecs];
#pragma unroll
			for (int j = 0; j < kVecs; j++) v[j] = *reinterpret_cast<const uint4*>(keys + base + ((size_t)j * kHistThreads + threadIdx.x) * 4);
#pragma unroll
			for (int j = 0; j < kVecs; j++) {
				histogram_add(lds, key_encode(v[j].x, kind), copy);
				histogram_add(lds, key_encode(v[j].y, kind), copy);
				histogram_add(lds, key_encode(v[j].z, kind), copy);
				histogram_add(lds, key_encode(v[j].w, kind), copy);
			}
		} else {
			for (int j = 0; j < kHistItems; j++) {
				const size_t i = base + (size_t)j * kHistThreads + threadIdx.x;
				if (i < n) histogram_add(lds, key_encode(keys[i], kind), copy);
			}
		}
	}
	__syncthreads();
	for (int i = threadIdx.x; i < 4 * kRadix; i += kHistThreads) {
		uint32_t c = 0;
#pragma unroll
		for (int k = 0; k < kHistCopies; k++) c += lds[i * kHistCopies + ((k + threadIdx.x) & (kHistCopies - 1))];  // rotated: no two lanes on one bank
		if (c) atomicAdd(&hist[i], c);
	}
}

// offsets[pass*256 + d] = number of keys whose pass-digit is < d. One group of 256 threads.
__global__ __launch_bounds__(kRadix) void radix_offsets_kernel(const uint32_t* __restrict__ hist, uint32_t* __restrict__ offsets) {
	__shared__ uint32_t wave_tot[4];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	for (int p = 0; p < 4; p++) {
		const uint32_t c = hist[p * kRadix + threadIdx.x];
		uint32_t incl = c;
#pragma unroll
		for (int off = 1; off < 64; off <<= 1) {
			uint32_t o = __shfl_up(incl, off, 64);
			if (lane >= off) incl += o;
		}
		if (lane == 63) wave_tot[wave] = incl;
		__syncthreads();
		uint32_t before = 0;
		for (int w = 0; w < wave; w++) before += wave_tot[w];
		offsets[p * kRadix + threadIdx.x] = before + incl - c;
		__syncthreads();
	}
}

// ---- 2. one pass --------------------------------------------------------------------------------

// WORDS: 32-bit words per element of the reorder buffer (1: keys alone, 2: key and payload side by side, so that a
// key-value tile changes places in one write and one read per element, between the same two barriers).
template <int WORDS>
struct alignas(16) OnesweepLds {
	uint32_t wave_hist[kRsWaves][kRadix];  // per-wave digit counts, then per-wave offsets within a digit
	uint32_t digit_start[kRadix];          // first tile-local position of each digit
	uint32_t bin_offset[kRadix];           // global position of a digit's first key of this tile, minus digit_start
	uint32_t exchange[kRsTile * WORDS];
	uint32_t scan_tmp[4];
	uint32_t tile;
};

// One 1024-thread group per compute unit (16384 keys and their payload: 128 KiB of reorder buffer; 109 registers per
// lane; ranks and tile positions are kept two to a register). With the same sixteen waves per unit as two 512-thread
// groups of 8192 keys, half as many tiles look back half as often and every digit's run in the scatter is twice as
// long: 2^28 keys + payload sort in 4.44-4.60 ms (58-60.5 Gkeys/s) instead of 5.0-5.35; a look-back window of 4 or 16
// tiles and a first look at the predecessors' words issued before the reorder leave that unchanged. The measurements
// below were made with the 512-thread tiles, 1.23 ms per pass: with the final stores removed a pass takes 0.94 ms, the same loads
// and stores with nothing in between (a copy) 0.71 ms; reading every tile's offsets from a finished run instead of
// looking back changes nothing, nor do 2 or 4 tiles per look-back step instead of 8, nor a quarter fewer vector
// instructions in the ranking; tiles of 4096 keys (runs of 64 B per digit in the scatter) are 40 % slower, three groups
// per compute unit at the price of 13 spilled registers 16 % slower. By time stamps at the phase boundaries a tile spends
// 9 % of its life loading keys, 8 % ranking, 17 % in the digit scan, 8 % in the reorder, 48 % between the start of its
// look-back and the barrier behind it, 10 % storing: the phases of a tile alternate between the memory system and the
// compute unit, and two tiles per compute unit do not keep both busy. More tiles per unit do not help either: with keys and
// payload taking turns in a one-word reorder buffer (43 KiB of group memory, the payload fetched after the key exchange,
// 80 registers without spills) three groups fit a compute unit and the sort takes 5.81 ms instead of 5.35; the same
// kernel held to two groups takes 5.60 ms (the price of the second exchange). Nor would splitting the pass into a counting
// kernel and a scattering kernel without any look-back: with the look-back replaced by the position uniform keys would have
// on average (wrong results, timing only) the sort takes 6.19 ms -- tiles then finish in no particular order, and the 512
// output streams (256 digits, keys and payload) advance less evenly than when the chain of prefixes paces them. Constant
// keys (one output stream) take 1.11 ms per pass.
template <bool HAS_VALUES, bool FULL>
__device__ __forceinline__ void radix_onesweep_body(
    OnesweepLds<HAS_VALUES ? 2 : 1>& s, const uint32_t tile, const uint32_t* __restrict__ keys_in, uint32_t* __restrict__ keys_out, const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ vals_out, size_t n, int shift,
    const uint32_t* __restrict__ digit_offsets, uint32_t* status, uint32_t* async_error, int kind, bool encode_on_load, bool decode_on_store) {
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const size_t base = (size_t)tile * kRsTile;
	// FULL: the whole tile lies inside the array, nothing below tests a bound
	const uint32_t valid_count = FULL ? (uint32_t)kRsTile : (uint32_t)(n - base);

	// Wave w owns tile-local keys [w*1024, (w+1)*1024); item j of lane l is key w*1024 + j*64 + l, so that
	// (j, lane) order is memory order. Keys past the end become 0xFFFFFFFF: digit 255 in every pass and
	// last in memory order, so they sort to the very end of the tile and are simply not written.
	uint32_t key[kRsItems];
	uint32_t val[kRsItems];
	const uint32_t first = wave * kRsWaveSpan + lane;
	const uint32_t* kp = keys_in + base + first;
	const uint32_t* vp = HAS_VALUES ? vals_in + base + first : nullptr;
#pragma unroll
	for (int j = 0; j < kRsItems; j++) {
		const bool valid = FULL || first + j * 64 < valid_count;
		uint32_t k = valid ? kp[j * 64] : 0xFFFFFFFFu;
		if (encode_on_load && valid) k = key_encode(k, kind);
		key[j] = k;
	}

	// Rank inside the wave: for every key, how many keys of this wave with the same digit precede it (< 1024: two
	// ranks share a register, item j in half j & 1 of word j / 2).
	uint32_t packed[kRsItems / 2];
#pragma unroll
	for (int j = 0; j < kRsItems; j++) {
		const uint32_t d = (key[j] >> shift) & 255u;
		// Which lanes hold the same digit: for every bit of the digit, the lanes whose bit differs from this lane's are
		// votes ^ mine (mine = the bit spread over a word); what no bit rules out is a peer. Written so that a bit costs
		// five vector instructions (sign-extending bit extract, compare = the ballot, two xor, half an or3 per half).
		uint32_t differ_lo = 0, differ_hi = 0;
#pragma unroll
		for (int b = 0; b < 8; b++) {
			const int32_t mine = __builtin_amdgcn_sbfe((int32_t)key[j], (uint32_t)(shift + b), 1u);  // 0 or -1
			const uint64_t votes = __ballot(mine != 0);
			differ_lo |= (uint32_t)votes ^ (uint32_t)mine;
			differ_hi |= (uint32_t)(votes >> 32) ^ (uint32_t)mine;
		}
		const uint64_t peers = ~(((uint64_t)differ_hi << 32) | differ_lo);
		const uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
		const uint32_t seen = s.wave_hist[wave][d];  // read by all peers before the first of them bumps it
		__builtin_amdgcn_wave_barrier();
		if (before == 0) s.wave_hist[wave][d] = seen + (uint32_t)__popcll(peers);
		__builtin_amdgcn_wave_barrier();
		const uint32_t rank = seen + before;
		if (j & 1)
			packed[j / 2] |= rank << 16;
		else
			packed[j / 2] = rank;
	}
	// The payload is fetched only now, so that it does not occupy registers during the ranking; it arrives while the
	// digits are scanned and the keys change places.
	if (HAS_VALUES) {
#pragma unroll
		for (int j = 0; j < kRsItems; j++) val[j] = (FULL || first + j * 64 < valid_count) ? vp[j * 64] : 0u;
	}
	__syncthreads();

	// Per digit: turn the per-wave counts into per-wave offsets, get the tile's count and publish it at once, so that
	// later tiles can add it up while this tile is still busy.
	uint32_t tile_count = 0, real_count = 0;
	uint32_t* my_status = status + (size_t)tile * kRadix + tid;
	if (tid < kRadix) {
		uint32_t run = 0;
#pragma unroll
		for (int w = 0; w < kRsWaves; w++) {
			const uint32_t c = s.wave_hist[w][tid];
			s.wave_hist[w][tid] = run;
			run += c;
		}
		tile_count = run;
		real_count = tile_count;
		if (tid == kRadix - 1) real_count -= (uint32_t)kRsTile - valid_count;  // padding is not data
		st_store(my_status, (tile == 0 ? kStPrefix : kStAggregate) | real_count);
		// exclusive scan of tile_count over the 256 digits (4 waves)
		uint32_t incl = tile_count;
#pragma unroll
		for (int off = 1; off < 64; off <<= 1) {
			uint32_t o = __shfl_up(incl, off, 64);
			if (lane >= off) incl += o;
		}
		if (lane == 63) s.scan_tmp[wave] = incl;
		s.digit_start[tid] = incl - tile_count;  // within this wave of digits; fixed up below
	}
	__syncthreads();
	if (tid < kRadix) {
		uint32_t before = 0;
		for (int w = 0; w < wave; w++) before += s.scan_tmp[w];
		const uint32_t start = s.digit_start[tid] + before;
		s.digit_start[tid] = start;
		// a key's tile position = its digit's first position + the keys of that digit in earlier waves + its rank in its
		// wave: the first two are folded into one table
#pragma unroll
		for (int w = 0; w < kRsWaves; w++) s.wave_hist[w][tid] += start;
	}
	__syncthreads();

	// Sort the tile by digit through LDS, keys then payload, back into registers in tile order. None of this needs
	// the global offsets, so the predecessors' status words have time to arrive before the look-back below.
#pragma unroll
	for (int j = 0; j < kRsItems; j++) {
		const uint32_t d = (key[j] >> shift) & 255u;
		const uint32_t rank = (j & 1) ? packed[j / 2] >> 16 : packed[j / 2] & 0xFFFFu;
		const uint32_t pos = s.wave_hist[wave][d] + rank;
		if (HAS_VALUES)
			*reinterpret_cast<uint2*>(&s.exchange[2 * pos]) = make_uint2(key[j], val[j]);
		else
			s.exchange[pos] = key[j];
	}
	__syncthreads();
#pragma unroll
	for (int j = 0; j < kRsItems; j++) {
		if (HAS_VALUES) {
			const uint2 kv = *reinterpret_cast<const uint2*>(&s.exchange[2 * (j * kRsThreads + tid)]);
			key[j] = kv.x;
			val[j] = kv.y;
		} else {
			key[j] = s.exchange[j * kRsThreads + tid];
		}
	}

	// Look back for the number of keys with this digit in all earlier tiles.
	if (tid < kRadix) {
		uint32_t exclusive = 0;
		if (tile > 0) {
			// Walk back over earlier tiles, kLookWindow of them per step: the status loads of a step are independent, so
			// their latencies overlap. Entries are consumed nearest first up to the first inclusive prefix; a tile that
			// has not published yet ends the step, and the walk resumes from it.
			int64_t look = (int64_t)tile - 1;
			uint32_t spins = 0;
			bool done = false;
			while (!done) {
				uint32_t st[kLookWindow];
#pragma unroll
				for (int i = 0; i < kLookWindow; i++) st[i] = look - i >= 0 ? st_load(status + (size_t)(look - i) * kRadix + tid) : kStPrefix;
				int used = 0;
#pragma unroll
				for (int i = 0; i < kLookWindow; i++) {
					const uint32_t flag = st[i] >> 30;
					if (!done && used == i && flag != 0) {
						exclusive += st[i] & kStValueMask;
						used = i + 1;
						done = flag == 2;
					}
				}
				look -= used;
				if (!done && used < kLookWindow) {
					if (++spins > kRsSpinLimit) {  // an earlier tile never published: give up and flag it
						*async_error = kAsyncErrLookbackTimeout;
						break;
					}
					__builtin_amdgcn_s_sleep(1);
				}
			}
			st_store(my_status, kStPrefix | ((exclusive + real_count) & kStValueMask));
		}
		s.bin_offset[tid] = digit_offsets[tid] + exclusive - s.digit_start[tid];
	}
	__syncthreads();

#pragma unroll
	for (int j = 0; j < kRsItems; j++) {
		const uint32_t p = j * kRsThreads + tid;
		uint32_t k = key[j];
		const uint32_t d = (k >> shift) & 255u;
		const uint32_t dst = s.bin_offset[d] + p;
		if (decode_on_store) k = key_decode(k, kind);
		if (FULL || p < valid_count) {
			// n < 2^30, so a byte offset fits 32 bits: one register per address beside the uniform base pointer
			const uint32_t at = dst << 2;
			*reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(keys_out) + at) = k;
			if (HAS_VALUES) *reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(vals_out) + at) = val[j];
		}
	}
}

template <bool HAS_VALUES>
__global__ __launch_bounds__(kRsThreads) void radix_onesweep_kernel(
    const uint32_t* __restrict__ keys_in, uint32_t* __restrict__ keys_out, const uint32_t* __restrict__ vals_in, uint32_t* __restrict__ vals_out, size_t n, int shift,
    const uint32_t* __restrict__ digit_offsets, uint32_t* status, uint32_t* ticket, uint32_t* async_error, int kind, bool encode_on_load, bool decode_on_store) {
	__shared__ OnesweepLds<HAS_VALUES ? 2 : 1> s;
	if (threadIdx.x == 0) s.tile = atomicAdd(ticket, 1u);
	for (int i = threadIdx.x; i < kRsWaves * kRadix; i += kRsThreads) (&s.wave_hist[0][0])[i] = 0;
	__syncthreads();
	const uint32_t tile = s.tile;
	if (((size_t)tile + 1) * kRsTile <= n)
		radix_onesweep_body<HAS_VALUES, true>(s, tile, keys_in, keys_out, vals_in, vals_out, n, shift, digit_offsets, status, async_error, kind, encode_on_load, decode_on_store);
	else
		radix_onesweep_body<HAS_VALUES, false>(s, tile, keys_in, keys_out, vals_in, vals_out, n, shift, digit_offsets, status, async_error, kind, encode_on_load, decode_on_store);
}

static int radix_sort_impl(int kind, const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                           uint32_t* keys_tmp, uint32_t* vals_tmp, size_t n) {
	State& st = state();
	// keys_out keeps the order-preserving unsigned form of the keys (what sort.py's own passes work on) when asked to
	const bool keep_mapped = (kind & TFHIP_KEY_KEEP_MAPPED) != 0;
	kind &= ~TFHIP_KEY_KEEP_MAPPED;
	if (n == 0) return TFHIP_OK;
	if (!keys_in || !keys_out) return fail(TFHIP_ERR_ARG, "null key pointer passed to the radix sort");
	if ((vals_in == nullptr) != (vals_out == nullptr)) return fail(TFHIP_ERR_ARG, "payload input and output must both be given or both be null");
	if (n >= ((size_t)1 << 30)) return fail(TFHIP_ERR_ARG, "radix sort supports fewer than 2^30 keys (got %zu)", n);
	if (kind < kKeyU32 || kind > kKeyF32) return fail(TFHIP_ERR_ARG, "unknown key kind %d", kind);
	if (keys_in == keys_out || (vals_in && vals_in == vals_out)) return fail(TFHIP_ERR_ARG, "radix sort is out of place: input and output must differ");
	{
		// Every pass scatters into one buffer while other tiles still read another: no two of the n-word buffers may overlap.
		const uint32_t* bufs[6] = {keys_in, keys_out, keys_tmp, vals_in, vals_out, vals_tmp};
		const char* names[6] = {"keys_in", "keys_out", "keys_tmp", "vals_in", "vals_out", "vals_tmp"};
		for (int a = 0; a < 6; a++)
			for (int b = a + 1; b < 6; b++) {
				if (!bufs[a] || !bufs[b]) continue;
				if (a == 0 && b == 3) continue;  // the two inputs are only read: one array may serve as keys and payload
				const uintptr_t pa = (uintptr_t)bufs[a], pb = (uintptr_t)bufs[b], bytes = n * sizeof(uint32_t);
				if (pa < pb + bytes && pb < pa + bytes)
					return fail(TFHIP_ERR_ARG, "radix sort buffers %s and %s overlap: keys_in, keys_out, keys_tmp, vals_in, vals_out and vals_tmp must be disjoint ranges of n words", names[a],
					            names[b]);
			}
	}
	const bool has_vals = vals_in != nullptr;
	const size_t tiles = (n + kRsTile - 1) / kRsTile;

	// scratch layout: [hist 4*256][offsets 4*256][tickets 4 (+pad to 16)][status 4 * tiles * 256][tmp keys n][tmp vals n]
	const size_t head_words = 4 * kRadix * 2 + 16;
	const size_t status_words = 4 * tiles * kRadix;
	size_t words = head_words + status_words;
	const size_t tmp_keys_at = (words + 63) & ~size_t(63);
	if (!keys_tmp) words = tmp_keys_at + n;
	const size_t tmp_vals_at = (words + 63) & ~size_t(63);
	if (has_vals && !vals_tmp) words = tmp_vals_at + n;
	uint32_t* base = (uint32_t*)scratch(words * sizeof(uint32_t));
	if (!base) return TFHIP_ERR_HIP;
	uint32_t* hist = base;
	uint32_t* offsets = base + 4 * kRadix;
	uint32_t* tickets = base + 8 * kRadix;
	uint32_t* status = base + head_words;
	if (!keys_tmp) keys_tmp = base + tmp_keys_at;
	if (has_vals && !vals_tmp) vals_tmp = base + tmp_vals_at;

	int rc = tfhip_fill_u32(base, 0u, head_words + status_words);
	if (rc) return rc;

	const size_t hist_tiles = (n + kHistTile - 1) / kHistTile;
	size_t hist_groups = hist_tiles < (size_t)st.compute_units * 2 ? hist_tiles : (size_t)st.compute_units * 2;  // 64 KiB of group memory each
	hipLaunchKernelGGL(radix_histogram_kernel, dim3((unsigned)hist_groups), dim3(kHistThreads), 0, st.stream, keys_in, n, hist, kind);
	TFHIP_CHECK_LAUNCH();
	hipLaunchKernelGGL(radix_offsets_kernel, dim3(1), dim3(kRadix), 0, st.stream, (const uint32_t*)hist, offsets);
	TFHIP_CHECK_LAUNCH();

	// in -> tmp -> out -> tmp -> out
	const uint32_t* src_k = keys_in;
	const uint32_t* src_v = vals_in;
	for (int pass = 0; pass < 4; pass++) {
		uint32_t* dst_k = (pass & 1) ? keys_out : keys_tmp;
		uint32_t* dst_v = (pass & 1) ? vals_out : vals_tmp;
		const bool enc = pass == 0 && kind != kKeyU32;
		const bool dec = pass == 3 && kind != kKeyU32 && !keep_mapped;
		if (has_vals)
			hipLaunchKernelGGL(radix_onesweep_kernel<true>, dim3((unsigned)tiles), dim3(kRsThreads), 0, st.stream, src_k, dst_k, src_v, dst_v, n, pass * 8,
			                   (const uint32_t*)(offsets + pass * kRadix), status + (size_t)pass * tiles * kRadix, tickets + pass, st.async_error_dev, kind, enc, dec);
		else
			hipLaunchKernelGGL(radix_onesweep_kernel<false>, dim3((unsigned)tiles), dim3(kRsThreads), 0, st.stream, src_k, dst_k, (const uint32_t*)nullptr,
			                   (uint32_t*)nullptr, n, pass * 8, (const uint32_t*)(offsets + pass * kRadix), status + (size_t)pass * tiles * kRadix, tickets + pass,
			                   st.async_error_dev, kind, enc, dec);
		TFHIP_CHECK_LAUNCH();
		src_k = dst_k;
		src_v = dst_v;
	}
	return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" {

int tfhip_radix_sort_kv(int key_kind, const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                        uint32_t* keys_tmp, uint32_t* vals_tmp, size_t n) {
	TFHIP_REQUIRE_INIT();
	return radix_sort_impl(key_kind, keys_in, vals_in, keys_out, vals_out, keys_tmp, vals_tmp, n);
}

int tfhip_radix_sort_kv_u32(const uint32_t* keys_in, const uint32_t* vals_in, uint32_t* keys_out, uint32_t* vals_out,
                            uint32_t* keys_tmp, uint32_t* vals_tmp, size_t n) {
	TFHIP_REQUIRE_INIT();
	return radix_sort_impl(kKeyU32, keys_in, vals_in, keys_out, vals_out, keys_tmp, vals_tmp, n);
}

}  // extern "C"
