#include "tf_backend.h"

#include <chrono>
#include <iostream>
#include <unordered_set>

#include "hip_generator.h"
#include "sort_composition.h"

namespace tfhost {

BackendType current_backend = BackendType::NotInitialized;
CodeGenLang current_kernel_lang = CodeGenLang::CPP;
std::string kernelCompileOptions;
KernelManager* global_kernel_manager = nullptr;

static void Check(int status, const std::string& what) {
	if (status != TFHIP_OK) throw std::runtime_error(what + ": " + tfhip_last_error());
}

// ---- kernel registry ----------------------------------------------------------------------------------

void KernelManager::AddKernelID(Program* program, Kernel* kernel) {
	programs.insert(program);
	kernel->kernel_id_ = global_kernel_id++;
	kernel_map[kernel->kernel_id_] = kernel;
}

void KernelManager::RemoveProgram(Program* program) {
	programs.erase(program);
	for (auto& k : program->kernels_) kernel_map.erase(k->kernel_id_);
}

void HipKernelManager::CompileKernel(Kernel* kernel) {
	if (!kernel->primitive.empty()) return;  // served by a precompiled primitive
	tfhip_kernel_t handle = nullptr;
	int status = tfhip_module_compile(kernel->full_generated_code_.c_str(), kernel->kernel_name_.c_str(), kernelCompileOptions.c_str(), &handle);
	if (status != TFHIP_OK) {
		// Same content as the GL backend's message: which kernel, the compiler's output, then the source
		// (Backends/OpenGL/KernelManager.h:79-83).
		throw std::runtime_error("Error compiling kernel " + std::to_string(kernel->kernel_id_) + "\n" + tfhip_last_error() + "\n" + kernel->full_generated_code_);
	}
	kernel_handles[kernel->kernel_id_] = handle;
	if (!kernel->scalar_entry.empty()) {
		tfhip_kernel_t scalar = nullptr;
		Check(tfhip_module_get_kernel(handle, kernel->scalar_entry.c_str(), &scalar), "Error loading kernel " + kernel->scalar_entry);
		scalar_handles[kernel->kernel_id_] = scalar;
	}
	if (compute_units == 0 && current_backend == BackendType::HIP) Check(tfhip_device_info(nullptr, 0, &compute_units, nullptr), "Failed to query the device");
}

// Kernels that stand for a whole reduction / scan / matmul / sort go to the hand-written primitives.
static void DispatchPrimitive(const Kernel* kernel, const TFDispatchInfo& info) {
	const std::string& p = kernel->primitive;
	const size_t n_tensors = info.read_write_count + info.read_only_count;
	if (n_tensors != kernel->primitive_tensors || info.variable_count != kernel->primitive_variables + 1)
		throw std::runtime_error("Primitive " + p + " expects " + std::to_string(kernel->primitive_tensors) + " tensors and " +
		                         std::to_string(kernel->primitive_variables) + " variables");
	auto buf = [&](size_t i) -> void* {
		const TFTensor& t = i < info.read_write_count ? info.read_write_tensors[i] : info.read_only_tensors[i - info.read_write_count];
		return ((TFHipBuffer*)t.buffer)->GetNative();
	};
	auto var = [&](size_t i) { return (size_t)info.variables[i]; };
	int status;
	if (p.rfind("sgemm_", 0) == 0) {
		// sgemm_<nn|nt|tn>[_<bias|bias_relu|mask_positive>]
		const std::string layout_name = p.substr(6, 2), tail = p.size() > 9 ? p.substr(9) : "";
		const int layout = layout_name == "nn" ? TFHIP_GEMM_NN : layout_name == "nt" ? TFHIP_GEMM_NT : layout_name == "tn" ? TFHIP_GEMM_TN : -1;
		const int epilogue = tail.empty() ? TFHIP_EPILOGUE_NONE : tail == "bias" ? TFHIP_EPILOGUE_BIAS : tail == "bias_relu" ? TFHIP_EPILOGUE_BIAS_RELU
		                     : tail == "mask_positive" ? TFHIP_EPILOGUE_MASK_POSITIVE : -1;
		if (layout < 0 || epilogue < 0 || n_tensors != (epilogue ? 4u : 3u)) throw std::runtime_error("Unknown primitive " + p);
		status = tfhip_sgemm_fused(layout, (const float*)buf(1), (const float*)buf(2), (float*)buf(0), var(0), var(1), var(2), epilogue,
		                           epilogue ? (const float*)buf(3) : nullptr);
	} else if (p.rfind("reduce_rows_", 0) == 0 || p.rfind("reduce_cols_", 0) == 0) {
		const std::string op = p.substr(12);
		const int code = op == "sum" ? TFHIP_REDUCE_SUM : op == "max" ? TFHIP_REDUCE_MAX : op == "min" ? TFHIP_REDUCE_MIN : -1;
		if (code < 0) throw std::runtime_error("Unknown primitive " + p);
		auto fn = p[7] == 'r' ? tfhip_reduce_rows_f32 : tfhip_reduce_cols_f32;
		status = fn(code, (const float*)buf(1), (float*)buf(0), var(0), var(1));
	} else if (p == "softmax_rows") {
		status = tfhip_softmax_rows_f32((const float*)buf(1), (float*)buf(0), var(0), var(1));
	} else if (p == "scan_u32" || p == "scan_i32") {
		status = tfhip_scan_inclusive_u32((const uint32_t*)buf(1), (uint32_t*)buf(0), var(0));
	} else if (p == "scan_f32") {
		status = tfhip_scan_inclusive_f32((const float*)buf(1), (float*)buf(0), var(0));
	} else if (p.rfind("radix_sort_kv_", 0) == 0) {
		const std::string kind = p.substr(14);
		const int code = kind == "u32" ? TFHIP_KEY_U32 : kind == "i32" ? TFHIP_KEY_I32 : kind == "f32" ? TFHIP_KEY_F32 : -1;
		if (code < 0) throw std::runtime_error("Unknown primitive " + p);
		status = tfhip_radix_sort_kv(code, (const uint32_t*)buf(4), (const uint32_t*)buf(5), (uint32_t*)buf(0), (uint32_t*)buf(1), (uint32_t*)buf(2), (uint32_t*)buf(3), var(0));
	} else {
		throw std::runtime_error("Unknown primitive " + p);
	}
	Check(status, "Primitive " + p + " failed");
}

// A kernel recognised as one lowered reduction / prefix-sum / matmul loop: evaluates its extents and strides
// for this dispatch and runs the primitive when the operands are dense. Returns false to fall back to the
// emitted kernel (which computes the same thing for any strides).
static bool TryDispatchIdiom(const Kernel* kernel, const TFDispatchInfo& info, HipKernelManager* manager) {
	const IdiomMatch& m = kernel->match;
	if (m.kind == IdiomMatch::None || m.kind == IdiomMatch::ExpSum || m.kind == IdiomMatch::Normalise || !manager->idioms_enabled) return false;
	const size_t n_tensors = info.read_write_count + info.read_only_count;
	if (n_tensors != kernel->read_write_memory.size() + kernel->read_only_memory.size()) return false;
	if (info.variable_count != kernel->variables.size() + 1 || info.variables[info.variable_count - 1] != 0) return false;
	auto buf = [&](int i) -> uint32_t* {
		const TFTensor& t = (size_t)i < info.read_write_count ? info.read_write_tensors[i] : info.read_only_tensors[i - info.read_write_count];
		return (uint32_t*)((TFHipBuffer*)t.buffer)->GetNative();
	};
	for (auto& c : m.conditions)
		if (c.first.Eval(info.variables) > c.second.Eval(info.variables)) return false;
	std::vector<long> d;
	for (const DimExpr& e : m.dims) d.push_back(e.Eval(info.variables));
	for (size_t i = 0; i < d.size(); i++)
		if (d[i] < (i < 2 ? 1 : 0)) return false;  // extents at least 1, strides never negative
	int status;
	if (m.kind == IdiomMatch::Reduce) {
		long T = d[0];
		const long K = d[1], in_t = d[2], in_k = d[3], out_t = d[4];
		const int code = m.op == "sum" ? TFHIP_REDUCE_SUM : m.op == "max" ? TFHIP_REDUCE_MAX : TFHIP_REDUCE_MIN;
		if (d.size() == 8) {
			// 2-D kernel (a reduction OptimizeReductions has split into chunks): outer index with extent T1
			const long T1 = d[5], in_t1 = d[6], out_t1 = d[7];
			if (T1 < 1) return false;
			if (in_k == 1 && in_t == K && in_t1 == T * K && out_t == 1 && out_t1 == T) {
				T *= T1;  // chunks of one row follow each other: [T1 * T] rows of K
			} else if (in_t == 1 && in_k == T && in_t1 == K * T && out_t == 1 && out_t1 == T) {
				// chunks of K rows under each other: one launch of the slab-wise column reduction
				Check(tfhip_reduce_cols_slabs_f32(code, (const float*)buf(m.buffers[1]), (float*)buf(m.buffers[0]), (size_t)(T1 * K), (size_t)T, (size_t)K),
				      "Primitive for kernel " + std::to_string(info.kernel_id) + " failed");
				return true;
			} else {
				return false;
			}
		}
		if (out_t != 1 && T != 1) return false;
		if ((in_k == 1 || K == 1) && (in_t == K || T == 1))
			status = tfhip_reduce_rows_f32(code, (const float*)buf(m.buffers[1]), (float*)buf(m.buffers[0]), (size_t)T, (size_t)K);
		else if ((in_t == 1 || T == 1) && (in_k == T || K == 1))
			status = tfhip_reduce_cols_f32(code, (const float*)buf(m.buffers[1]), (float*)buf(m.buffers[0]), (size_t)K, (size_t)T);
		else
			return false;
	} else if (m.kind == IdiomMatch::Scan) {
		const long T = d[0], K = d[1], in_t = d[2], in_k = d[3], out_t = d[4], out_k = d[5];
		const uint32_t* in = buf(m.buffers[1]);
		uint32_t* out = buf(m.buffers[0]);
		const bool is_float = m.type == TFType_Float;
		long batch = 1, in_b = 0, out_b = 0;  // outer thread index of a 2-D kernel
		if (d.size() == 9) {
			batch = d[6];
			in_b = d[7];
			out_b = d[8];
			if (batch < 1) return false;
		}
		const bool same = in_t == out_t && in_k == out_k && in_b == out_b;
		if (same && in_k == 1 && (T == 1 || in_t == K) && (batch == 1 || in_b == T * K)) {
			// lines that follow each other in memory, each scanned along its own contiguous axis
			status = is_float ? tfhip_scan_inclusive_rows_f32((const float*)in, (float*)out, (size_t)(T * batch), (size_t)K)
			                  : tfhip_scan_inclusive_rows_u32(in, out, (size_t)(T * batch), (size_t)K);
		} else if (same && in_t == 1 && in_k == T && (batch == 1 || in_b == T * K)) {
			// down the columns of [K, T] matrices that follow each other
			status = is_float ? tfhip_scan_inclusive_cols_f32((const float*)in, (float*)out, (size_t)batch, (size_t)K, (size_t)T)
			                  : tfhip_scan_inclusive_cols_u32(in, out, (size_t)batch, (size_t)K, (size_t)T);
		} else {
			return false;
		}
	} else {
		if (m.op == "tail") {
			const long N = d[0], M = d[1], K = d[2], a_i = d[3], a_k = d[4], b_k = d[5], b_j = d[6];
			if (K < 1 || kernel->tail_kernel == nullptr) return false;
			const bool a_plain = (a_k == 1 || K == 1) && (a_i == K || M == 1);
			const bool a_transposed = (a_i == 1 || M == 1) && (a_k == M || K == 1);
			const bool b_plain = (b_j == 1 || N == 1) && (b_k == N || K == 1);
			const bool b_transposed = (b_k == 1 || K == 1) && (b_j == K || N == 1);
			const int layout = a_plain && b_plain ? TFHIP_GEMM_NN : a_plain && b_transposed ? TFHIP_GEMM_NT : a_transposed && b_plain ? TFHIP_GEMM_TN : -1;
			if (layout < 0) return false;
			// product[M, N] in a pooled temporary; the stream's order lets the pool hand it on right after the launch
			TFTensor* product = global_memory_manager->AllocateTensor({(size_t)M, (size_t)N}, TFDataFormat{TFType_Float, 32}, "matmul_product");
			try {
				Check(tfhip_sgemm_fused(layout, (const float*)buf(m.buffers[1]), (const float*)buf(m.buffers[2]), (float*)((TFHipBuffer*)product->buffer)->GetNative(),
				                        (size_t)M, (size_t)N, (size_t)K, TFHIP_EPILOGUE_NONE, nullptr),
				      "Primitive for kernel " + std::to_string(info.kernel_id) + " failed");
				std::vector<TFTensor> tensors;
				for (size_t i = 0; i < info.read_write_count; i++) tensors.push_back(info.read_write_tensors[i]);
				for (size_t i = 0; i < info.read_only_count; i++) tensors.push_back(info.read_only_tensors[i]);
				tensors.push_back(*product);
				TFDispatchInfo tail = info;
				tail.kernel_id = kernel->tail_kernel->kernel_id_;
				tail.read_write_count = tensors.size();
				tail.read_write_tensors = tensors.data();
				tail.read_only_count = 0;
				tail.read_only_tensors = nullptr;
				manager->DispatchNow(tail);
				manager->dispatch_count--;  // the pair counts as the one dispatch the host issued
			} catch (...) {
				global_memory_manager->DeallocateTensor(*product);
				throw;
			}
			global_memory_manager->DeallocateTensor(*product);
			return true;
		}
		const long N = d[0], M = d[1], K = d[2], a_i = d[3], a_k = d[4], b_k = d[5], b_j = d[6], c_i = d[7], c_j = d[8];
		if (K < 1 || (c_j != 1 && N != 1) || (c_i != N && M != 1)) return false;
		const bool a_plain = (a_k == 1 || K == 1) && (a_i == K || M == 1);
		const bool a_transposed = (a_i == 1 || M == 1) && (a_k == M || K == 1);
		const bool b_plain = (b_j == 1 || N == 1) && (b_k == N || K == 1);
		const bool b_transposed = (b_k == 1 || K == 1) && (b_j == K || N == 1);
		const float* A = (const float*)buf(m.buffers[1]);
		const float* B = (const float*)buf(m.buffers[2]);
		float* C = (float*)buf(m.buffers[0]);
		const int epilogue = m.op.empty() ? TFHIP_EPILOGUE_NONE : m.op == "bias" ? TFHIP_EPILOGUE_BIAS : m.op == "bias_relu" ? TFHIP_EPILOGUE_BIAS_RELU : TFHIP_EPILOGUE_MASK_POSITIVE;
		const float* aux = epilogue ? (const float*)buf(m.buffers[3]) : nullptr;
		const int layout = a_plain && b_plain ? TFHIP_GEMM_NN : a_plain && b_transposed ? TFHIP_GEMM_NT : a_transposed && b_plain ? TFHIP_GEMM_TN : -1;
		if (layout < 0) return false;
		if (d.size() == 13) {
			// batched: d[9] products, matrix t of A / B / C starts d[10] / d[11] / d[12] words after matrix t - 1
			const long T = d[9], a_t = d[10], b_t = d[11], c_t = d[12];
			if (T < 1 || T > 65535 || c_t < M * N || (a_t != 0 && a_t < M * K) || (b_t != 0 && b_t < K * N)) return false;
			status = tfhip_sgemm_batched(layout, A, B, C, (size_t)M, (size_t)N, (size_t)K, (size_t)T, (size_t)a_t, (size_t)b_t, (size_t)c_t);
		} else {
			status = tfhip_sgemm_fused(layout, A, B, C, (size_t)M, (size_t)N, (size_t)K, epilogue, aux);
		}
	}
	Check(status, "Primitive for kernel " + std::to_string(info.kernel_id) + " failed");
	return true;
}

// ---- chains of dispatches ---------------------------------------------------------------------------------------

void HipKernelManager::RefreshOptions() { idioms_enabled = std::getenv("TFHIP_NO_IDIOMS") == nullptr; }

void HipKernelManager::Hold(const TFDispatchInfo& info) { HoldInto(chain.dispatches, info); }

void HipKernelManager::HoldInto(std::vector<Deferred>& list, const TFDispatchInfo& info) {
	list.emplace_back();
	Deferred& d = list.back();
	d.tensors.assign(info.read_write_tensors, info.read_write_tensors + info.read_write_count);
	d.tensors.insert(d.tensors.end(), info.read_only_tensors, info.read_only_tensors + info.read_only_count);
	d.variables.assign(info.variables, info.variables + info.variable_count);
	d.info = info;  // the pointers are set when it runs: the vectors may still move
}

// A split reduction whose two stages are held and whose chunk tensor the program has released: one call of the
// reduction primitive on the original matrix. Returns false when that is not the state of the chain.
bool HipKernelManager::RunSplitReductionWhole() {
	if (chain.dispatches.size() != 2 || !chain.chunk_max || !chain.row_max || chain.chunk_sum || chain.row_sum) return false;
	bool released = false;
	for (const TFTensor& t : chain.frees) released |= t.buffer == chain.chunk_max;
	if (!released) return false;
	auto ptr = [](TFBuffer* b) { return (float*)((TFHipBuffer*)b)->GetNative(); };
	const int code = chain.op == "sum" ? TFHIP_REDUCE_SUM : chain.op == "max" ? TFHIP_REDUCE_MAX : TFHIP_REDUCE_MIN;
	Check((chain.down ? tfhip_reduce_cols_f32 : tfhip_reduce_rows_f32)(code, ptr(chain.x), ptr(chain.row_max), (size_t)chain.rows, (size_t)chain.cols),
	      "Primitive for the kernels up to " + std::to_string(chain.dispatches.back().info.kernel_id) + " failed");
	dispatch_count += 2;
	idiom_dispatch_count += 2;
	fused_chain_count++;
	chain.dispatches.clear();
	return true;
}

// Row maxima and row sums of exp(x - max) are both held (two to four dispatches) and the next thing is not the
// normalising kernel: a log-softmax, a cross-entropy, ... One call computes both statistics from one read of x.
bool HipKernelManager::RunSoftmaxStatistics() {
	if (chain.stage != 4 || !chain.row_max || !chain.row_sum) return false;
	for (TFBuffer* chunk : {chain.chunk_max, chain.chunk_sum}) {
		if (!chunk) continue;
		bool released = false;
		for (const TFTensor& t : chain.frees) released |= t.buffer == chunk;
		if (!released) return false;
	}
	auto ptr = [](TFBuffer* b) { return (float*)((TFHipBuffer*)b)->GetNative(); };
	Check(tfhip_softmax_rows_stats_f32(ptr(chain.x), nullptr, ptr(chain.row_max), ptr(chain.row_sum), (size_t)chain.rows, (size_t)chain.cols),
	      "Primitive for the kernels up to " + std::to_string(chain.dispatches.back().info.kernel_id) + " failed");
	dispatch_count += chain.dispatches.size();
	idiom_dispatch_count += chain.dispatches.size();
	fused_chain_count++;
	chain.dispatches.clear();
	return true;
}

void HipKernelManager::DeferFree(TFTensor tensor) {
	if (sort.state != SortRegion::Idle) {
		sort.frees.push_back(tensor);
		if (sort.state == SortRegion::Closed && SortRegionReleased()) RunSortRegion();
		return;
	}
	chain.frees.push_back(tensor);
	// a complete split reduction only waited to learn that nobody reads its chunk results
	if (chain.stage == 5 && tensor.buffer == chain.chunk_max) FlushDeferred();
}

void HipKernelManager::RunHeld(std::vector<Deferred>& dispatches, std::vector<TFTensor>& frees, std::exception_ptr error) {
	for (Deferred& d : dispatches) {
		if (error) break;
		TFDispatchInfo info = d.info;
		info.read_write_tensors = d.tensors.data();
		info.read_only_tensors = d.tensors.data() + info.read_write_count;
		info.variables = d.variables.data();
		try {
			DispatchNow(info);
		} catch (...) {
			error = std::current_exception();
		}
	}
	for (TFTensor& t : frees) global_memory_manager->DeallocateTensor(t);
	if (error) std::rethrow_exception(error);
}

void HipKernelManager::FlushDeferred() {
	if (sort.state == SortRegion::Closed && SortRegionReleased())
		RunSortRegion();
	else if (sort.state != SortRegion::Idle)
		AbandonSortRegion();
	if (chain.stage == 0 && chain.frees.empty()) return;
	DispatchChain held;
	std::exception_ptr error;
	try {
		if (chain.stage == 5 || chain.stage == 2) RunSplitReductionWhole();
		if (chain.stage == 4) RunSoftmaxStatistics();
	} catch (...) {
		error = std::current_exception();
		chain.dispatches.clear();
	}
	held = std::move(chain);
	chain = DispatchChain();
	RunHeld(held.dispatches, held.frees, error);
}

// True when the dispatch opened or continued the chain (it is then held back, or the whole chain has just run).
bool HipKernelManager::AdvanceChain(const Kernel* kernel, const TFDispatchInfo& info) {
	const IdiomMatch& m = kernel->match;
	if (m.kind != IdiomMatch::Reduce && m.kind != IdiomMatch::ExpSum && m.kind != IdiomMatch::Normalise) return false;
	if (m.type != TFType_Float || !idioms_enabled) return false;
	const size_t n_tensors = info.read_write_count + info.read_only_count;
	if (n_tensors != kernel->read_write_memory.size() + kernel->read_only_memory.size()) return false;
	if (info.variable_count != kernel->variables.size() + 1 || info.variables[info.variable_count - 1] != 0) return false;
	for (auto& c : m.conditions)
		if (c.first.Eval(info.variables) > c.second.Eval(info.variables)) return false;
	std::vector<long> d;
	for (const DimExpr& e : m.dims) d.push_back(e.Eval(info.variables));
	auto buffer = [&](int i) -> TFBuffer* {
		return ((size_t)i < info.read_write_count ? info.read_write_tensors[i] : info.read_only_tensors[i - info.read_write_count]).buffer;
	};
	// A reduction-shaped kernel (Reduce, ExpSum) over a dense matrix, along the rows: whole rows ([rows] threads, `cols`
	// steps) or, split, chunks ([rows, chunks] threads, `chunk` steps, chunks * chunk == cols; chunks == 0 for whole
	// rows). Or down the columns (`down`): whole columns ([cols] threads, `rows` steps) or slabs ([slabs, cols] threads,
	// `slab` steps, slabs * slab == rows; the slab count is then in `chunks`).
	long rows = 0, cols = 0, chunks = 0;
	bool down = false;
	const bool reduction_shaped = m.kind != IdiomMatch::Normalise;
	const bool outer = reduction_shaped && (d.size() == 8 || d.size() == 11);
	if (reduction_shaped) {
		const long T = d[0], K = d[1], in_t = d[2], in_k = d[3], out_t = d[4];
		if (T < 1 || K < 1) return false;
		if (outer) {
			const long T1 = d[5], in_t1 = d[6], out_t1 = d[7];
			if (T1 < 1 || out_t != 1 || out_t1 != T) return false;
			if (in_k == 1 && in_t == K && in_t1 == T * K) {
				rows = T1, cols = T * K, chunks = T;
			} else if (m.kind == IdiomMatch::Reduce && in_t == 1 && in_k == T && in_t1 == K * T) {
				down = true, rows = T1 * K, cols = T, chunks = T1;
			} else {
				return false;
			}
		} else if (in_k == 1 && in_t == K && out_t == 1) {
			rows = T, cols = K;
		} else if (m.kind == IdiomMatch::Reduce && in_t == 1 && in_k == T && out_t == 1 && chain.stage == 1 && chain.down) {
			down = true, rows = K, cols = T;  // only as the second stage of a split reduction down the columns
		} else {
			return false;
		}
	}
	TFBuffer* out = buffer(m.buffers[0]);
	TFBuffer* in = buffer(m.buffers[1]);
	switch (chain.stage) {
		case 0:
			// opens a chain: the first stage of a split reduction (any operation, either axis), or whole-row maxima
			if (m.kind != IdiomMatch::Reduce || in == out) return false;
			if (!chunks && (down || m.op != "max")) return false;
			chain.x = in;
			chain.rows = rows;
			chain.cols = cols;
			chain.op = m.op;
			chain.down = down;
			chain.chunks = chunks;
			(chunks ? chain.chunk_max : chain.row_max) = out;
			chain.stage = chunks ? 1 : 2;
			Hold(info);
			return true;
		case 1:  // the second stage: the same operation over the chunk (slab) results
			if (m.kind != IdiomMatch::Reduce || m.op != chain.op || chunks || down != chain.down || in != chain.chunk_max || out == chain.x || out == in) return false;
			if (down ? (cols != chain.cols || rows != chain.chunks) : (rows != chain.rows || cols != chain.chunks)) return false;
			chain.row_max = out;
			// row maxima may be the start of a softmax; anything else is complete and waits for the release of the chunk tensor
			chain.stage = (!down && m.op == "max") ? 2 : 5;
			Hold(info);
			return true;
		case 2: {  // sums of exp(x - max): whole rows or chunks
			if (m.kind != IdiomMatch::ExpSum || down || in != chain.x || buffer(m.buffers[2]) != chain.row_max || rows != chain.rows || cols != chain.cols) return false;
			if (out == chain.x || out == chain.row_max) return false;
			// the maximum is addressed by the row alone
			const size_t at = outer ? 8 : 5;
			if (outer ? !(d[at] == 0 && d[at + 1] == 0 && d[at + 2] == 1) : !(d[at] == 1 && d[at + 1] == 0)) return false;
			(chunks ? chain.chunk_sum : chain.row_sum) = out;
			chain.sum_chunks = chunks;
			chain.stage = chunks ? 3 : 4;
			Hold(info);
			return true;
		}
		case 3:  // row sums from the chunk sums
			if (m.kind != IdiomMatch::Reduce || m.op != "sum" || chunks || down || in != chain.chunk_sum || rows != chain.rows || cols != chain.sum_chunks) return false;
			if (out == chain.x || out == chain.row_max || out == in) return false;
			chain.row_sum = out;
			chain.stage = 4;
			Hold(info);
			return true;
		case 4: {
			if (m.kind != IdiomMatch::Normalise) return false;
			TFBuffer* y = out;
			if (in != chain.x || buffer(m.buffers[2]) != chain.row_max || buffer(m.buffers[3]) != chain.row_sum) return false;
			if (y == chain.x || y == chain.row_max || y == chain.row_sum) return false;
			const long C = d[0], R = d[1];
			if (C != chain.cols || R != chain.rows) return false;
			// X and Y dense row-major, maxima and sums one word per row
			if (d[2] != 1 || d[3] != C || d[4] != 1 || d[5] != C || d[6] != 0 || d[7] != 1 || d[8] != 0 || d[9] != 1) return false;
			// the chunk tensors are not written: the program must have released them already
			for (TFBuffer* chunk : {chain.chunk_max, chain.chunk_sum}) {
				if (!chunk) continue;
				bool released = false;
				for (const TFTensor& t : chain.frees) released |= t.buffer == chunk;
				if (!released || chunk == y) return false;
			}
			auto ptr = [](TFBuffer* b) { return (float*)((TFHipBuffer*)b)->GetNative(); };
			Check(tfhip_softmax_rows_stats_f32(ptr(chain.x), ptr(y), ptr(chain.row_max), ptr(chain.row_sum), (size_t)R, (size_t)C),
			      "Primitive for the kernels up to " + std::to_string(info.kernel_id) + " failed");
			const size_t served = chain.dispatches.size() + 1;
			dispatch_count += served;
			idiom_dispatch_count += served;
			fused_chain_count++;
			chain.dispatches.clear();
			chain.stage = 0;
			FlushDeferred();  // the frees
			return true;
		}
	}
	return false;
}

void HipKernelManager::DispatchKernel(TFDispatchInfo info) {
	Kernel* kernel = GetKernel(info.kernel_id);
	if (sort.state == SortRegion::Following && FollowSortDispatch(kernel, info)) return;
	if (sort.state != SortRegion::Idle) FlushDeferred();  // not the composition (or the region is over): what is held runs first
	if (kernel != nullptr && kernel->primitive.empty() && kernel->match.kind != IdiomMatch::None) {
		if (AdvanceChain(kernel, info)) return;
		if (HasDeferredWork()) {
			// not the chain's next kernel: what is held back runs first; this dispatch may then open a chain of its own
			FlushDeferred();
			if (AdvanceChain(kernel, info)) return;
		}
	} else {
		FlushDeferred();
	}
	DispatchNow(info);
}

void HipKernelManager::DispatchNow(TFDispatchInfo info) {
	Kernel* kernel = GetKernel(info.kernel_id);
	if (kernel != nullptr && !kernel->primitive.empty()) {
		DispatchPrimitive(kernel, info);
		dispatch_count++;
		return;
	}
	if (kernel != nullptr && TryDispatchIdiom(kernel, info, this)) {
		dispatch_count++;
		idiom_dispatch_count++;
		return;
	}
	if (kernel != nullptr && kernel->dense_variant != nullptr) {
		// enough threads to fill every SIMD several times over: the thread-serial form of the loops
		std::vector<int> g = kernel->group_size;
		while (g.size() < 3) g.push_back(1);
		const uint64_t logical = (uint64_t)info.work_group_count * g[0] * g[1] * g[2];
		if (logical >= (uint64_t)compute_units * 4096) {
			TFDispatchInfo dense = info;
			dense.kernel_id = kernel->dense_variant->kernel_id_;
			DispatchNow(dense);
			return;
		}
	}
	auto it = kernel_handles.find(info.kernel_id);
	if (it == kernel_handles.end() || kernel == nullptr) throw std::runtime_error("Kernel " + std::to_string(info.kernel_id) + " was not compiled");
	if (info.read_write_count == 0) throw std::runtime_error("No tensors provided to kernel");

	// Generated hosts pass every tensor in read_write_tensors (rw first, then ro) and none in
	// read_only_tensors (CPP.cpp:485-491); accept the split form too.
	void* buffers[64];
	size_t n_buffers = 0;
	const size_t expected = kernel->read_write_memory.size() + kernel->read_only_memory.size();
	if (info.read_write_count + info.read_only_count != expected)
		throw std::runtime_error("Kernel " + std::to_string(info.kernel_id) + " expects " + std::to_string(expected) + " tensors, got " +
		                         std::to_string(info.read_write_count + info.read_only_count));
	if (expected > 64) throw std::runtime_error("Too many tensors bound to one kernel");
	for (size_t i = 0; i < info.read_write_count; i++) buffers[n_buffers++] = ((TFHipBuffer*)info.read_write_tensors[i].buffer)->GetNative();
	for (size_t i = 0; i < info.read_only_count; i++) buffers[n_buffers++] = ((TFHipBuffer*)info.read_only_tensors[i].buffer)->GetNative();

	// Variable block: the host's words (user scalars + block offset) followed by the group count.
	const size_t expected_vars = kernel->variables.size() + 1;
	if (info.variable_count != expected_vars)
		throw std::runtime_error("Kernel " + std::to_string(info.kernel_id) + " expects " + std::to_string(expected_vars) + " variable words, got " + std::to_string(info.variable_count));
	if (info.work_group_count > 0xFFFFFFFFull) throw std::runtime_error("work_group_count does not fit 32 bits");
	uint32_t vars[258];
	if (expected_vars + 1 > 258) throw std::runtime_error("Too many kernel variables");
	for (size_t i = 0; i < info.variable_count; i++) vars[i] = info.variables[i];
	vars[info.variable_count] = (uint32_t)info.work_group_count;

	std::vector<int> group = kernel->group_size;
	while (group.size() < 3) group.push_back(1);
	uint64_t grid;
	uint32_t bx = (uint32_t)kernel->hip_threads, by = 1, bz = 1;
	tfhip_kernel_t handle = it->second;
	if (kernel->idiom == "group") {
		grid = info.work_group_count;
		bx = group[0];
		by = group[1];
		bz = group[2];
	} else if (kernel->idiom == "reduction:wave") {
		const uint64_t logical = (uint64_t)info.work_group_count * group[0] * group[1] * group[2];
		const uint64_t per_block = 256 / (uint64_t)kernel->lanes_per_thread;
		grid = (logical + per_block - 1) / per_block;
	} else if (kernel->idiom == "reduction:block") {
		const uint64_t logical = (uint64_t)info.work_group_count * group[0] * group[1] * group[2];
		grid = (logical + 63) / 64;
	} else {
		// "flat" and "flat:vec4": Q IR groups per tile; the grid is padded to a multiple of 8 because the
		// kernels deal tiles to the 8 dies in contiguous bands (surplus groups exit at once).
		const uint64_t logical = (uint64_t)info.work_group_count * group[0] * group[1] * group[2];
		auto scalar = scalar_handles.find(info.kernel_id);
		if (kernel->idiom == "flat:vec4" && scalar != scalar_handles.end() && logical < (uint64_t)compute_units * 1024) {
			// Fewer than one 256-thread group of quads per compute unit: run one logical thread per lane instead.
			handle = scalar->second;
			bx = (uint32_t)kernel->scalar_hip_threads;
			grid = (info.work_group_count + kernel->scalar_groups_per_hip_block - 1) / kernel->scalar_groups_per_hip_block;
		} else {
			grid = (info.work_group_count + kernel->groups_per_hip_block - 1) / kernel->groups_per_hip_block;
			grid *= kernel->hip_blocks_per_tile;
		}
		grid = (grid + 7) / 8 * 8;
	}
	if (grid > 0x7FFFFFFFull) throw std::runtime_error("Dispatch of kernel " + std::to_string(info.kernel_id) + " needs " + std::to_string(grid) + " groups, more than one launch can hold");
	Check(tfhip_launch(handle, (uint32_t)grid, bx, by, bz, buffers, n_buffers, vars, info.variable_count + 1), "Failed to dispatch kernel " + std::to_string(info.kernel_id));
	dispatch_count++;
}

void HipKernelManager::FreeKernel(size_t kernel_id) {
	auto sc = scalar_handles.find(kernel_id);
	if (sc != scalar_handles.end()) {
		tfhip_module_unload(sc->second);
		scalar_handles.erase(sc);
	}
	auto it = kernel_handles.find(kernel_id);
	if (it == kernel_handles.end()) return;
	tfhip_module_unload(it->second);
	kernel_handles.erase(it);
}

void HipKernelManager::FreeAllKernels() {
	for (auto& kv : scalar_handles) tfhip_module_unload(kv.second);
	scalar_handles.clear();
	for (auto& kv : kernel_handles) tfhip_module_unload(kv.second);
	kernel_handles.clear();
}

// ---- code generation and compilation ---------------------------------------------------------------------

void GenerateKernel(Program* program, Kernel* kernel) {
	switch (current_kernel_lang) {
		case CodeGenLang::HIP:
			GenerateHIPKernel(program, kernel);
			return;
		default:
			throw std::runtime_error("Code generation for this language is not implemented yet");
	}
}

void GenerateCode(Program* program) {
	if (global_kernel_manager == nullptr) throw std::runtime_error("Backend not initialized");
	const size_t count = program->kernels_.size();  // tail kernels are appended while this runs
	for (size_t i = 0; i < count; i++) {
		Kernel* kernel = program->kernels_[i].get();
		global_kernel_manager->AddKernelID(program, kernel);
		kernel->kernel_name_ = "kernel_" + std::to_string(kernel->kernel_id_);
		if (!kernel->primitive.empty()) continue;
		kernel->sort_role = (int)SortRoleOf(kernel);  // before the emitter annotates the tree
		GenerateKernel(program, kernel);
		if (current_kernel_lang != CodeGenLang::HIP) continue;
		if (kernel->wants_dense_variant) {
			Kernel* dense = CloneKernel(program, kernel);
			dense->serial_loops = true;
			global_kernel_manager->AddKernelID(program, dense);
			dense->kernel_name_ = "kernel_" + std::to_string(dense->kernel_id_);
			GenerateKernel(program, dense);
			kernel->dense_variant = dense;
		}
		MatchKernelIdiom(kernel);
		if (kernel->match.kind == IdiomMatch::Matmul && kernel->match.op == "tail") {
			// A matmul loop with an element-wise tail of its own: the kernel without the loop becomes a second
			// kernel that reads the product of the matmul primitive.
			Kernel* tail = MakeMatmulTailKernel(program, kernel, kernel->match.accumulator, kernel->match.loop);
			global_kernel_manager->AddKernelID(program, tail);
			tail->kernel_name_ = "kernel_" + std::to_string(tail->kernel_id_);
			GenerateKernel(program, tail);
			kernel->tail_kernel = tail;
		}
	}
}

void CompileKernels(Program* program) {
	auto start = std::chrono::high_resolution_clock::now();
	for (auto& kernel : program->kernels_) {
		switch (current_backend) {
			case BackendType::HIP:
			case BackendType::CodeGen:  // no device: hiprtc still checks that the source builds for gfx950
				((HipKernelManager*)global_kernel_manager)->CompileKernel(kernel.get());
				break;
			default:
				throw std::runtime_error("Backend not implemented");
		}
	}
	auto end = std::chrono::high_resolution_clock::now();
	program->shader_compile_time = std::chrono::duration<float, std::milli>(end - start).count();
}

// ---- backend lifetime ---------------------------------------------------------------------------------

void StopBackend() {
	if (current_backend == BackendType::NotInitialized) return;
	delete global_kernel_manager;
	global_kernel_manager = nullptr;
	delete global_memory_manager;
	global_memory_manager = nullptr;
	if (current_backend == BackendType::HIP) tfhip_shutdown();
	current_backend = BackendType::NotInitialized;
}

void InitializeBackend(BackendType type, const std::string& compiler_options, CodeGenLang kernel_lang) {
	if (current_backend != BackendType::NotInitialized) {
		std::cout << "Warning: Backend already initialized, stopping current backend\n" << std::endl;
		StopBackend();
	}
	kernelCompileOptions = compiler_options;  // non-CPU backends default to no extra options (Backend.cpp:27-37)
	switch (type) {
		case BackendType::HIP:
			Check(tfhip_init(0), "Failed to initialize the HIP backend");
			current_kernel_lang = CodeGenLang::HIP;
			global_memory_manager = new HipMemoryManager();
			global_kernel_manager = new HipKernelManager();
			break;
		case BackendType::CodeGen:
			// Emits and hiprtc-checks source without a device; programs cannot be executed.
			current_kernel_lang = CodeGenLang::HIP;
			global_memory_manager = nullptr;
			global_kernel_manager = new HipKernelManager();
			break;
		default:
			throw std::runtime_error("Backend not implemented");
	}
	current_backend = type;
	if (kernel_lang != CodeGenLang::None) current_kernel_lang = kernel_lang;
}

void Finish() {
	if (current_backend == BackendType::HIP) Check(tfhip_sync(), "Failed to synchronize");
}

// ---- runtime callbacks (Backend.cpp:96-133) ---------------------------------------------------------------

static TFTensor Allocator(const char* name, const size_t* a, size_t dim, TFDataFormat format, void*) {
	try {
		std::vector<size_t> shape(a, a + dim);
		return *global_memory_manager->AllocateTensor(shape, format, name);
	} catch (const std::exception& e) {
		size_t size = 1;
		for (size_t i = 0; i < dim; i++) size *= a[i];
		throw std::runtime_error("Error allocating tensor " + std::string(name) + ": " + e.what() + ", requested size: " + std::to_string(size));
	}
}

static HipKernelManager* HipManager() { return current_backend == BackendType::HIP ? (HipKernelManager*)global_kernel_manager : nullptr; }

static void Deallocator(TFTensor a, void*) {
	HipKernelManager* km = HipManager();
	if (km && km->HasDeferredWork())
		km->DeferFree(a);  // a dispatch that is held back may still name this buffer
	else
		global_memory_manager->DeallocateTensor(a);
}
static uint32_t Readback(TFTensor a, size_t index, void*) {
	if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	return global_memory_manager->ReadbackValue(&a, index);
}
static void Writeback(TFTensor a, size_t index, uint32_t value, void*) {
	if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	global_memory_manager->WritebackValue(&a, index, value);
}
static void Dispatch(TFDispatchInfo info, void*) { global_kernel_manager->DispatchKernel(info); }
static void Region(const char* name, bool begin, void*) {
	if (current_backend == BackendType::HIP) {
		((HipKernelManager*)global_kernel_manager)->OnRegion(name, begin);
		if (begin)
			tfhip_range_push(name);
		else
			tfhip_range_pop();
	}
}

TFRuntime GetRuntimeCallbacks() { return TFRuntime{Allocator, Deallocator, Readback, Writeback, Dispatch, Region, nullptr}; }

std::vector<TFTensor*> ExecuteProgram(Program* program, std::vector<TFTensor*> inputs) {
	if (current_backend == BackendType::CodeGen) throw std::runtime_error("Cannot execute program with code generation backend");
	if (current_backend == BackendType::NotInitialized) throw std::runtime_error("Backend not initialized");
	if ((size_t)program->input_count != inputs.size())
		throw std::runtime_error("Invalid number of inputs for TensorProgram. Expected " + std::to_string(program->input_count) + ", got " + std::to_string(inputs.size()));

	std::vector<TFTensor> input_tensors;
	for (TFTensor* t : inputs) input_tensors.push_back(*t);
	TFTensor* out = new TFTensor[program->output_count];  // kept alive for the wrappers of the outputs
	try {
		if (HipKernelManager* km = HipManager()) km->RefreshOptions();
		program->execute_callback(input_tensors.data(), out, GetRuntimeCallbacks());
		if (HipKernelManager* km = HipManager()) km->FlushDeferred();
	} catch (const std::exception& e) {
		delete[] out;
		try {
			if (HipKernelManager* km = HipManager()) km->FlushDeferred();
		} catch (...) {
		}
		throw std::runtime_error("Error executing program " + program->program_name + ": " + e.what());
	}
	std::vector<TFTensor*> outputs(program->output_count);
	for (int i = 0; i < program->output_count; i++) outputs[i] = &out[i];
	return outputs;
}

// ---- recorded programs ----------------------------------------------------------------------------------------

static void* DevicePointer(const TFTensor* t) { return ((TFHipBuffer*)t->buffer)->GetNative(); }

RecordedProgram* RecordProgram(Program* program, std::vector<TFTensor*> inputs, size_t repeat, const std::vector<int>& feedback) {
	if (current_backend != BackendType::HIP) throw std::runtime_error("Programs can only be recorded on the HIP backend");
	if (repeat == 0) throw std::runtime_error("Cannot record zero executions");
	if (repeat > 1 && feedback.empty()) throw std::runtime_error("Recording more than one execution needs feedback (outputs feeding the next inputs)");
	if (!feedback.empty() && feedback.size() != inputs.size())
		throw std::runtime_error("Feedback has " + std::to_string(feedback.size()) + " entries for " + std::to_string(inputs.size()) + " inputs");
	for (int f : feedback)
		if (f < -1 || f >= program->output_count) throw std::runtime_error("Feedback names output " + std::to_string(f) + " of " + std::to_string(program->output_count));

	// The ordinary run: loads modules, sizes the scratch buffer and fills the pool with buffers of the right sizes.
	std::vector<TFTensor*> first = ExecuteProgram(program, inputs);
	auto is_input = [&](const TFTensor* t) {
		for (TFTensor* in : inputs)
			if (in->buffer == t->buffer) return true;
		return false;
	};
	auto release_all = [&](const std::vector<TFTensor*>& tensors, const std::vector<TFTensor*>& keep) {
		std::unordered_set<TFBuffer*> done;
		for (TFTensor* t : keep) done.insert(t->buffer);
		for (TFTensor* t : tensors) {
			if (is_input(t) || !done.insert(t->buffer).second) continue;
			global_memory_manager->DeallocateTensor(*t);
		}
	};
	for (size_t i = 0; i < feedback.size(); i++) {
		if (feedback[i] < 0) continue;
		const TFTensor* from = first[feedback[i]];
		if (GetShape(from) != GetShape(inputs[i]) || from->format.type != inputs[i]->format.type) {
			release_all(first, {});
			throw std::runtime_error("Feedback: output " + std::to_string(feedback[i]) + " and input " + std::to_string(i) + " differ in shape or type");
		}
	}
	release_all(first, {});

	RecordedProgram* recorded = new RecordedProgram();
	global_memory_manager->BeginHold();
	bool recording = false;
	try {
		Check(tfhip_graph_begin(), "Failed to start recording");
		recording = true;
		std::vector<TFTensor*> current = inputs, out;
		for (size_t r = 0; r < repeat; r++) {
			std::vector<TFTensor*> previous = out;
			out = ExecuteProgram(program, current);
			// The previous execution's outputs have been consumed; the stream's order makes their reuse safe.
			release_all(previous, out);
			for (size_t i = 0; i < feedback.size(); i++)
				if (feedback[i] >= 0) current[i] = out[feedback[i]];
		}
		for (size_t i = 0; i < feedback.size(); i++) {
			if (feedback[i] < 0 || out[feedback[i]]->buffer == inputs[i]->buffer) continue;
			Check(tfhip_d2d(DevicePointer(inputs[i]), DevicePointer(out[feedback[i]]), GetSize(inputs[i])), "Failed to record the feedback copy");
		}
		recording = false;
		Check(tfhip_graph_end(&recorded->graph), "Failed to finish recording");
		recorded->outputs = out;
	} catch (...) {
		if (recording) tfhip_graph_end(nullptr);
		global_memory_manager->EndHold(false);
		delete recorded;
		throw;
	}
	recorded->buffers = global_memory_manager->EndHold(true);
	tfhip_graph_node_count(recorded->graph, &recorded->nodes);
	return recorded;
}

void ReplayProgram(RecordedProgram* recorded) { Check(tfhip_graph_launch(recorded->graph), "Failed to replay"); }

void DestroyRecordedProgram(RecordedProgram* recorded) {
	if (!recorded) return;
	tfhip_graph_destroy(recorded->graph);  // waits for the stream
	if (global_memory_manager) global_memory_manager->Unreserve(recorded->buffers);
	delete recorded;
}

}  // namespace tfhost
