// The `Radix sort` region of tf.sort.radix, followed dispatch by dispatch and served by one onesweep sort.
//
// What arrives between region_begin('Radix sort') and region_end('Radix sort') (Python/TensorFrost/sort.py:74-176):
//   keys = tf.copy(keys) [fused with map_float_to_uint / map_int_to_uint]; values = tf.copy(values)        :78-87
//   keys1 / values1 = tf.buffer(...)                                                                      :96-100
//   iters // 2 host-loop iterations, each two SortIteration calls on swapped buffers                      :102-174
//     region 'Radix sort iteration' { histogram, unpack, chunk sums, chunk scan, scan in chunks, totals, scatter }
// With the default bits_per_pass = 6 and max_bits = 32 that is 6 passes: the result is the stable ascending order of
// the whole 32-bit (mapped) key and lies in the buffers the prologue wrote. The onesweep sort gives exactly that order
// in 4 passes of 8 bits, so one call replaces the region when -- and only when -- everything seen is that composition.
#include <algorithm>

#include "HIP.h"

namespace TFSHIM_NAMESPACE {

using tfhip::kSortGroup;
using tfhip::kSortScanChunk;
using tfhip::SortRole;

namespace {

const TFTensor& TensorAt(const TFDispatchInfo& info, size_t i) { return i < info.read_write_count ? info.read_write_tensors[i] : info.read_only_tensors[i - info.read_write_count]; }

}  // namespace

void HipKernelManager::OnRegion(const char* name_c, bool begin) {
	const std::string name = name_c ? name_c : "";
	if (sort.state == SortRegion::Idle) {
		if (begin && name == "Radix sort" && idioms_enabled) {
			FlushChain();  // a chain of another kind that is still held runs first
			sort = SortRegion();
			sort.state = SortRegion::Following;
		}
		return;
	}
	if (sort.state == SortRegion::Closed) {  // anything but the releases it waits for settles it
		FlushChain();
		if (begin && name == "Radix sort") OnRegion(name_c, begin);
		return;
	}
	bool fits = false;
	if (name == "Radix sort iteration") {
		if (begin) {
			fits = !sort.in_iteration && sort.step == 0 && sort.iterations == sort.passes && !sort.copies.empty();
			sort.in_iteration = true;
			sort.iterations++;
		} else {
			fits = sort.in_iteration && sort.step == 0 && sort.iterations == sort.passes;
			sort.in_iteration = false;
		}
	} else if (name == "Radix sort" && !begin) {
		// 6 passes of 6 bits cover the 32 bits of a key: fewer (max_bits < 31) sort by the low bits only
		if (!sort.in_iteration && sort.passes == 6) {
			sort.state = SortRegion::Closed;
			if (SortRegionReleased()) RunSortRegion();
			return;
		}
	}
	if (!fits) AbandonSortRegion();
}

bool HipKernelManager::FollowSortDispatch(const HipKernelInfo* kernel, const TFDispatchInfo& info) {
	if (kernel == nullptr || kernel->sort_role == 0) return false;
	const SortRole role = (SortRole)kernel->sort_role;
	const size_t n_tensors = info.read_write_count + info.read_only_count;
	if (n_tensors != kernel->tensor_count) return false;
	if (info.variable_count != kernel->variable_count + 1 || info.variables[info.variable_count - 1] != 0) return false;
	auto buffer = [&](size_t i) { return TensorAt(info, i).buffer; };
	auto var = [&](size_t i) { return (long)(int)info.variables[i]; };
	SortRegion& s = sort;
	auto known = [&](TFBuffer* b) {
		if (b == s.keys[0] || b == s.keys[1] || b == s.values[0] || b == s.values[1]) return true;
		for (auto& c : s.copies)
			if (b == c.dst || b == c.src) return true;
		return std::find(s.intermediates.begin(), s.intermediates.end(), b) != s.intermediates.end();
	};
	// a buffer no earlier dispatch of the region has named: the result of an allocation of this pass
	auto fresh = [&](TFBuffer* b) {
		if (b == nullptr || known(b)) return false;
		s.intermediates.push_back(b);
		return true;
	};

	if (!s.in_iteration) {
		// the prologue: copies of the caller's keys (mapped to uint when they are float or int) and values
		if (s.passes != 0 || s.iterations != 0) return false;
		if (role != SortRole::Copy && role != SortRole::MapFloat && role != SortRole::MapInt) return false;
		const long n = var(0);
		if (n < 1 || n >= (1l << 30) || (s.N != 0 && n != s.N)) return false;
		TFBuffer *dst = buffer(0), *src = buffer(1);
		if (dst == src || s.copies.size() >= 2) return false;
		for (auto& c : s.copies)
			if (c.dst == dst || c.dst == src || c.src == dst) return false;
		if (dst->size < (size_t)n || src->size < (size_t)n) return false;
		s.N = n;
		s.G = (n + kSortGroup - 1) / kSortGroup;
		s.chunks = (s.G + kSortScanChunk - 1) / kSortScanChunk;
		s.copies.push_back({dst, src, (int)role});
		HoldInto(s.dispatches, info);
		return true;
	}

	const int pass = s.passes;
	const int from = pass & 1, to = from ^ 1;
	switch (s.step) {
		case 0: {
			if (role != SortRole::Histogram || var(0) != s.N || var(1) != s.G || var(2) != pass) return false;
			TFBuffer* k_in = buffer(1);
			if (pass == 0) {
				bool copied = false;
				for (auto& c : s.copies) copied |= c.dst == k_in;
				if (!copied) return false;
				s.keys[0] = k_in;
			} else if (k_in != s.keys[from]) {
				return false;
			}
			if (!fresh(buffer(0))) return false;
			s.packed = buffer(0);
			break;
		}
		case 1:
			if (role != SortRole::Unpack || var(0) != s.G || buffer(1) != s.packed || !fresh(buffer(0))) return false;
			s.hist = buffer(0);
			break;
		case 2:
			if (role != SortRole::ChunkSums || var(0) != s.G || var(1) != s.chunks || buffer(1) != s.hist || !fresh(buffer(0))) return false;
			s.sums = buffer(0);
			break;
		case 3:
			if (role != SortRole::ChunkScan || var(0) != s.chunks || buffer(1) != s.sums || !fresh(buffer(0))) return false;
			s.sums_scanned = buffer(0);
			break;
		case 4:
			if (role != SortRole::ScanInChunks || var(0) != s.G || var(1) != s.chunks || buffer(1) != s.hist || buffer(2) != s.sums_scanned || !fresh(buffer(0))) return false;
			s.scan = buffer(0);
			break;
		case 5:
			if (role != SortRole::Totals || var(0) != s.G || buffer(1) != s.scan || !fresh(buffer(0))) return false;
			s.total = buffer(0);
			break;
		case 6: {
			if (role != SortRole::Scatter && role != SortRole::ScatterKeys) return false;
			const bool with_values = role == SortRole::Scatter;
			if (var(0) != s.N || var(1) != s.G || var(2) != pass) return false;
			TFBuffer* k_out = buffer(0);
			TFBuffer* v_out = with_values ? buffer(1) : nullptr;
			const size_t ro = with_values ? 2 : 1;
			TFBuffer* k_in = buffer(ro);
			TFBuffer* v_in = with_values ? buffer(ro + 1) : nullptr;
			if (buffer(n_tensors - 2) != s.scan || buffer(n_tensors - 1) != s.total || k_in != s.keys[from]) return false;
			if (pass == 0) {
				s.has_values = with_values;
				if (s.copies.size() != (with_values ? 2u : 1u)) return false;
				if (with_values) {
					// the values are a plain copy of the caller's
					bool copied = false;
					for (auto& c : s.copies) copied |= c.dst == v_in && c.dst != s.keys[0] && c.role == (int)SortRole::Copy;
					if (!copied) return false;
					s.values[0] = v_in;
				}
				if (known(k_out) || (with_values && (known(v_out) || v_out == k_out))) return false;
				if (k_out->size < (size_t)s.N || (with_values && v_out->size < (size_t)s.N)) return false;
				s.keys[1] = k_out;
				s.values[1] = v_out;
			} else {
				if (with_values != s.has_values || k_out != s.keys[to]) return false;
				if (with_values && (v_in != s.values[from] || v_out != s.values[to])) return false;
			}
			break;
		}
		default: return false;
	}
	HoldInto(s.dispatches, info);
	if (++s.step == 7) {
		s.step = 0;
		s.passes++;
	}
	return true;
}

bool HipKernelManager::SortRegionReleased() const {
	auto released = [&](TFBuffer* b) {
		for (const TFTensor& t : sort.frees)
			if (t.buffer == b) return true;
		return false;
	};
	// nobody can read what the skipped kernels would have written
	for (TFBuffer* b : sort.intermediates)
		if (!released(b)) return false;
	if (!released(sort.keys[1])) return false;
	if (sort.has_values && !released(sort.values[1])) return false;
	// the results themselves are alive, and not handed out twice
	return !released(sort.keys[0]) && !(sort.has_values && released(sort.values[0]));
}

void HipKernelManager::RunSortRegion() {
	SortRegion s = std::move(sort);
	sort = SortRegion();
	const SortRegion::Copy* key_copy = nullptr;
	const SortRegion::Copy* value_copy = nullptr;
	for (auto& c : s.copies) {
		if (c.dst == s.keys[0]) key_copy = &c;
		if (s.has_values && c.dst == s.values[0]) value_copy = &c;
	}
	std::exception_ptr error;
	if (key_copy == nullptr || (s.has_values && value_copy == nullptr)) {
		RunHeld(s.dispatches, s.frees, error);
		return;
	}
	const int kind = key_copy->role == (int)SortRole::MapFloat ? (TFHIP_KEY_F32 | TFHIP_KEY_KEEP_MAPPED)
	                 : key_copy->role == (int)SortRole::MapInt ? (TFHIP_KEY_I32 | TFHIP_KEY_KEEP_MAPPED)
	                                                            : TFHIP_KEY_U32;
	auto ptr = [](TFBuffer* b) { return b ? (uint32_t*)((TFHipBuffer*)b)->GetNative() : nullptr; };
	try {
		FlushBatch();  // gathered small dispatches were issued before the region's
		if (tfhip_radix_sort_kv(kind, ptr(key_copy->src), s.has_values ? ptr(value_copy->src) : nullptr, ptr(s.keys[0]), ptr(s.values[0]), ptr(s.keys[1]), ptr(s.values[1]),
		                        (size_t)s.N) != TFHIP_OK)
			throw std::runtime_error(std::string("Primitive for the region 'Radix sort' failed: ") + tfhip_last_error());
		dispatch_count += s.dispatches.size();
		idiom_dispatch_count += s.dispatches.size();
		fused_chain_count++;
	} catch (...) {
		error = std::current_exception();
	}
	s.dispatches.clear();
	RunHeld(s.dispatches, s.frees, error);
}

void HipKernelManager::AbandonSortRegion() {
	SortRegion s = std::move(sort);
	sort = SortRegion();
	RunHeld(s.dispatches, s.frees, nullptr);
}

}  // namespace TFSHIM_NAMESPACE
