// The `Radix sort` region of tf.sort.radix, held back, checked as a whole and served by one onesweep sort.
//
// What arrives between region_begin('Radix sort') and region_end('Radix sort') (Python/TensorFrost/sort.py:74-176):
//   keys = tf.copy(keys) [with map_float_to_uint / map_int_to_uint]; values = tf.copy(values)               :78-87
//   keys1 / values1 = tf.buffer(...)                                                                      :96-100
//   iters // 2 host-loop iterations, each two SortIteration calls on swapped buffers                      :102-174
//     region 'Radix sort iteration' { group histograms, their prefix sums over groups and digits, scatter }
// How many kernels that is, and what each of them contains, is the compiler's decision (Compiler/Graph/Scope.cpp:5-35
// fuses adjacent element-wise operations of one shape; element-wise values may be recomputed inside the kernels that
// load them). So nothing here counts kernels or compares them with templates. The region is served when its data flow
// and the few computations its result depends on -- found per kernel by the code generator, see SortFeatures in
// hip_kernel_info.h -- show that it is a least-significant-digit radix sort over all 32 key bits:
// each pass a stable partition by the next digit is what the scatter kernel does GIVEN the group / digit offsets it
// reads, and those come from kernels that see nothing but that pass's keys. The onesweep sort produces the same
// stable order in 4 passes of 8 bits.
#include <algorithm>

#include "HIP.h"

namespace TFSHIM_NAMESPACE {

namespace {

TFBuffer* BufferOf(const std::vector<TFTensor>& tensors, int i) { return i >= 0 && (size_t)i < tensors.size() ? tensors[(size_t)i].buffer : nullptr; }

bool Contains(const std::vector<TFBuffer*>& list, const TFBuffer* b) { return std::find(list.begin(), list.end(), b) != list.end(); }

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
			fits = !sort.in_iteration && !sort.dispatches.empty();
			sort.in_iteration = true;
			sort.iterations++;
		} else {
			fits = sort.in_iteration && !sort.iteration_of.empty() && sort.iteration_of.back() == sort.iterations - 1;
			sort.in_iteration = false;
		}
	} else if (name == "Radix sort" && !begin) {
		if (!sort.in_iteration && ValidateSortRegion()) {
			sort.state = SortRegion::Closed;
			if (SortRegionReleased()) RunSortRegion();
			return;
		}
	}
	if (!fits) AbandonSortRegion();
}

bool HipKernelManager::FollowSortDispatch(const HipKernelInfo* kernel, const TFDispatchInfo& info) {
	// Only emitted kernels are understood: their bindings say what they read and write.
	if (kernel == nullptr || !kernel->primitive.empty()) return false;
	// (the host passes every tensor in the read-write list, written ones first, as the generated host program does:
	// Backend/CodeGen/Langs/CPP.cpp:485-491; which of them the kernel writes is the kernel's own knowledge)
	if (info.read_write_count + info.read_only_count != kernel->tensor_count) return false;
	if (info.variable_count != kernel->variable_count + 1 || info.variables[info.variable_count - 1] != 0) return false;
	// sort.py dispatches nothing between two iterations or behind the last one
	if (!sort.in_iteration && sort.iterations != 0) return false;
	HoldInto(sort.dispatches, info);
	sort.iteration_of.push_back(sort.in_iteration ? sort.iterations - 1 : -1);
	sort.kernel_of.push_back(kernel);
	return true;
}

bool HipKernelManager::ValidateSortRegion() {
	SortRegion& s = sort;
	const int passes = s.iterations;
	if (passes < 1 || s.dispatches.size() != s.iteration_of.size()) return false;

	// The scatter that ends every iteration: buffers, digit, element count.
	struct Pass {
		size_t scatter = 0;  // index of the dispatch
		TFBuffer *keys_in = nullptr, *values_in = nullptr, *keys_out = nullptr, *values_out = nullptr;
		long shift = 0, n = 0;
		uint32_t mask = 0;
	};
	std::vector<Pass> pass((size_t)passes);
	std::vector<bool> seen((size_t)passes, false);
	for (size_t d = 0; d < s.dispatches.size(); d++) {
		const int it = s.iteration_of[d];
		if (it < 0) continue;
		if (it >= passes) return false;
		pass[(size_t)it].scatter = d;  // the last dispatch of the iteration
		seen[(size_t)it] = true;
	}
	for (int p = 0; p < passes; p++) {
		if (!seen[(size_t)p]) return false;
		Pass& ps = pass[(size_t)p];
		const auto& f = s.kernel_of[ps.scatter]->sort;
		const Deferred& d = s.dispatches[ps.scatter];
		if (!f.scatter) return false;
		ps.keys_in = BufferOf(d.tensors, f.keys_in);
		ps.keys_out = BufferOf(d.tensors, f.keys_out);
		ps.values_in = BufferOf(d.tensors, f.values_in);
		ps.values_out = BufferOf(d.tensors, f.values_out);
		ps.shift = f.scatter_shift.Eval(d.variables.data());
		ps.n = f.scatter_n.Eval(d.variables.data());
		ps.mask = f.scatter_mask;
		if (!ps.keys_in || !ps.keys_out || (ps.values_in == nullptr) != (ps.values_out == nullptr)) return false;
	}
	const bool has_values = pass[0].values_in != nullptr;
	const long n = pass[0].n;
	const uint32_t mask = pass[0].mask;
	int bits = 0;
	while (bits < 32 && (mask >> bits) != 0) bits++;
	if (n < 1 || n >= (1l << 30) || bits < 1 || bits > 16 || mask != (bits == 32 ? 0xFFFFFFFFu : (1u << bits) - 1u)) return false;
	if ((long)passes * bits < 32) return false;  // fewer bits than a key has: the region sorts by the low bits only
	for (int p = 0; p < passes; p++) {
		const Pass& ps = pass[(size_t)p];
		if (ps.n != n || ps.mask != mask || ps.shift != (long)p * bits || ps.shift > 31) return false;
		if ((ps.values_in != nullptr) != has_values) return false;
		// a ping-pong pair: a pass reads what the one before wrote and writes what that one read
		if (p > 0) {
			const Pass& before = pass[(size_t)p - 1];
			if (ps.keys_in != before.keys_out || ps.keys_out != before.keys_in) return false;
			if (has_values && (ps.values_in != before.values_out || ps.values_out != before.values_in)) return false;
		}
	}
	TFBuffer* chain[4] = {pass[0].keys_in, pass[0].keys_out, pass[0].values_in, pass[0].values_out};
	for (int i = 0; i < 4; i++) {
		if (chain[i] == nullptr) continue;
		if (chain[i]->size < (size_t)n) return false;
		for (int j = 0; j < i; j++)
			if (chain[i] == chain[j]) return false;
	}
	auto in_chain = [&](const TFBuffer* b) { return b == chain[0] || b == chain[1] || b == chain[2] || b == chain[3]; };

	// Before the first iteration: element-wise copies that make the first pass's keys and values from buffers of the caller.
	TFBuffer *source_keys = nullptr, *source_values = nullptr;
	int key_map = -1;
	for (size_t d = 0; d < s.dispatches.size(); d++) {
		if (s.iteration_of[d] != -1) continue;
		const auto& f = s.kernel_of[d]->sort;
		const Deferred& held = s.dispatches[d];
		if (!f.copies_only || f.copies.empty()) return false;
		for (const auto& c : f.copies) {
			TFBuffer *dst = BufferOf(held.tensors, c.dst), *src = BufferOf(held.tensors, c.src);
			if (!dst || !src || c.extent.Eval(held.variables.data()) != n || src->size < (size_t)n) return false;
			if (dst == pass[0].keys_in && !source_keys && c.map >= 0 && c.map <= 2) {
				source_keys = src;
				key_map = c.map;
			} else if (has_values && dst == pass[0].values_in && !source_values && c.map == 0) {
				source_values = src;
			} else {
				return false;  // a copy sort.py does not make
			}
		}
	}
	if (!source_keys || (has_values && !source_values)) return false;
	if (in_chain(source_keys) || (has_values && in_chain(source_values))) return false;

	// Every other kernel of an iteration: sees only this pass's keys / values and what the iteration has written so far,
	// writes outside the chain; one of them takes this pass's digit of the keys.
	std::vector<TFBuffer*> intermediates;
	for (int p = 0; p < passes; p++) {
		const Pass& ps = pass[(size_t)p];
		std::vector<TFBuffer*> written;
		bool digit_taken = false;
		for (size_t d = 0; d < s.dispatches.size(); d++) {
			if (s.iteration_of[d] != p) continue;
			const Deferred& held = s.dispatches[d];
			const HipKernelInfo* k = s.kernel_of[d];
			const size_t rw = k->read_write_count;
			if (d == ps.scatter) {
				// its tables come from this iteration
				for (size_t i = rw; i < held.tensors.size(); i++) {
					TFBuffer* b = held.tensors[i].buffer;
					if (b != ps.keys_in && b != ps.values_in && !Contains(written, b)) return false;
				}
				continue;
			}
			for (size_t i = rw; i < held.tensors.size(); i++) {
				TFBuffer* b = held.tensors[i].buffer;
				if (b != ps.keys_in && b != ps.values_in && !Contains(written, b)) return false;
			}
			for (size_t i = 0; i < rw; i++) {
				TFBuffer* b = held.tensors[i].buffer;
				if (in_chain(b) || b == source_keys || b == source_values) return false;
				if (!Contains(written, b)) written.push_back(b);
			}
			for (const auto& g : k->sort.digits)
				if (BufferOf(held.tensors, g.keys) == ps.keys_in && g.mask == mask && g.shift.Eval(held.variables.data()) == ps.shift) digit_taken = true;
		}
		if (!digit_taken) return false;
		for (TFBuffer* b : written) {
			if (Contains(intermediates, b)) return false;  // deallocations are held back, so no buffer serves two iterations
			intermediates.push_back(b);
		}
	}

	const Pass& last = pass[(size_t)passes - 1];
	s.N = n;
	s.has_values = has_values;
	s.key_kind = key_map == 1 ? (TFHIP_KEY_F32 | TFHIP_KEY_KEEP_MAPPED) : key_map == 2 ? (TFHIP_KEY_I32 | TFHIP_KEY_KEEP_MAPPED) : TFHIP_KEY_U32;
	s.source_keys = source_keys;
	s.source_values = source_values;
	s.result_keys = last.keys_out;
	s.result_values = last.values_out;
	s.other_keys = last.keys_in;
	s.other_values = last.values_in;
	s.intermediates = std::move(intermediates);
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
	if (!released(sort.other_keys)) return false;
	if (sort.has_values && !released(sort.other_values)) return false;
	// the results themselves are alive, and not handed out twice
	return !released(sort.result_keys) && !(sort.has_values && released(sort.result_values));
}

void HipKernelManager::RunSortRegion() {
	SortRegion s = std::move(sort);
	sort = SortRegion();
	std::exception_ptr error;
	auto ptr = [](TFBuffer* b) { return b ? (uint32_t*)((TFHipBuffer*)b)->GetNative() : nullptr; };
	try {
		FlushBatch();  // gathered small dispatches were issued before the region's
		if (tfhip_radix_sort_kv(s.key_kind, ptr(s.source_keys), s.has_values ? ptr(s.source_values) : nullptr, ptr(s.result_keys), ptr(s.result_values), ptr(s.other_keys),
		                        ptr(s.other_values), (size_t)s.N) != TFHIP_OK)
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
