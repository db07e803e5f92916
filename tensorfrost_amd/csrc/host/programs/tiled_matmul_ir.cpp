// The reference's hand-tiled matrix product (examples/Algorithms/matrix_mul.ipynb, cell 0, "2d local + group tiled
// version") in IR form: a user kernel `tf.kernel([N / 4, K / 4], group_size=[16, 16])` with two group buffers of
// 64 x 64 floats, two barriers per 64-wide panel and a 4 x 4 block of results per thread. Nothing here names a
// primitive and the kernel is not one matmul loop, so it is emitted as written (group mapping).
//
//   A[N, M] x B[M, K] -> C[N, K].  The panel loop runs over the contracted dimension M (the example's text bounds it
//   by K, which is the same number for the square matrices it is run on). Loads and stores use the clamped index
//   mode of user indexing (Compiler/Steps/GraphOps.cpp:989-1043). N, M and K must be multiples of 64, as in the
//   example's own run (4096): a thread outside the kernel's shape loads no tile elements, so a ragged group would
//   leave holes in the tiles its neighbours read, and a clamped column of a ragged last panel would be added twice.
#include "registry.h"

namespace tfhost {

static void BuildTiledMatmulIr(Program* program, const std::vector<int64_t>&) {
	constexpr int BK = 64, TBK = 4, GK = BK / TBK;
	KernelBuilder kb(program, 2, {GK, GK});
	// c + v as the reference's constant folding leaves it: 0 + v is v itself
	auto offset = [&](int c, V v) { return c == 0 ? v : kb.Const(c) + v; };
	V C = kb.Buffer("C", false), A = kb.Buffer("A", true), B = kb.Buffer("B", true);
	V N = kb.Var("N", TFType_Int), M = kb.Var("M", TFType_Int), K = kb.Var("K", TFType_Int);
	V Kq = kb.Named(K / kb.Const(TBK), "vdiv"), Nq = kb.Named(N / kb.Const(TBK), "vdiv");
	std::vector<V> idx = kb.ThreadIndices({Kq, Nq});
	V j = idx[0], i = idx[1];
	V A_tile = kb.GroupMemory("A_group_tile", TFType_Float, BK * BK);
	V B_tile = kb.GroupMemory("B_group_tile", TFType_Float, BK * BK);
	V tx = kb.Named(kb.BlockThreadId(1), "tx"), ty = kb.Named(kb.BlockThreadId(0), "ty");
	V gx = kb.Named(i - tx, "gx"), gy = kb.Named(j - ty, "gy");
	auto at = [&](V row, V col, V rows, V cols) {
		return kb.Clamp(row, kb.Const(0), rows - kb.Const(1)) * cols + kb.Clamp(col, kb.Const(0), cols - kb.Const(1));
	};
	std::vector<V> results;
	for (int r = 0; r < TBK * TBK; r++) results.push_back(kb.Accumulator("result", TFType_Float, FloatBits(0.0f)));

	kb.Loop(kb.Const(0), M, kb.Const(BK), [&](V blk) {
		for (int blk_ty = 0; blk_ty < TBK; blk_ty++)
			for (int blk_tx = 0; blk_tx < TBK; blk_tx++) {
				V ltx = offset(blk_tx * GK, tx), lty = offset(blk_ty * GK, ty);
				kb.Store(A_tile, ltx * kb.Const(BK) + lty, kb.Load(A, at(kb.Const(TBK) * gx + ltx, blk + lty, N, M), TFType_Float));
			}
		for (int blk_tx = 0; blk_tx < TBK; blk_tx++)
			for (int blk_ty = 0; blk_ty < TBK; blk_ty++) {
				V ltx = offset(blk_tx * GK, tx), lty = offset(blk_ty * GK, ty);
				kb.Store(B_tile, ltx * kb.Const(BK) + lty, kb.Load(B, at(blk + ltx, kb.Const(TBK) * gy + lty, M, K), TFType_Float));
			}
		kb.Barrier();
		kb.Loop(kb.Const(0), kb.Const(BK), kb.Const(1), [&](V k) {
			V b_row[TBK];
			for (int tid = 0; tid < TBK; tid++) b_row[tid] = kb.Load(B_tile, k * kb.Const(BK) + (offset(tid * GK, ty)), TFType_Float);
			for (int tid = 0; tid < TBK; tid++) {
				V a_value = kb.Load(A_tile, (offset(tid * GK, tx)) * kb.Const(BK) + k, TFType_Float);
				for (int tid2 = 0; tid2 < TBK; tid2++) kb.Set(results[tid * TBK + tid2], results[tid * TBK + tid2] + a_value * b_row[tid2]);
			}
		});
		kb.Barrier();
	});
	for (int tid = 0; tid < TBK; tid++)
		for (int tid2 = 0; tid2 < TBK; tid2++) {
			V ltx = offset(tid * GK, tx), lty = offset(tid2 * GK, ty);
			kb.Store(C, at(kb.Const(TBK) * gx + ltx, kb.Const(TBK) * gy + lty, N, K), results[tid * TBK + tid2]);
		}
	Kernel* kernel = kb.Finish();

	HostBuilder h(program);
	V A_in = h.Input("A", {-1, -1}, TFType_Float);
	V rows = h.Shape(A_in)[0], inner = h.Shape(A_in)[1];
	V B_in = h.Input("B", {inner, -1}, TFType_Float);
	V cols = h.Shape(B_in)[1];
	auto tiles = [&](V extent) { return extent % h.Const(64) == h.Const(0); };
	h.AssertValue("tiled_matmul_ir: every dimension must be a multiple of 64", (tiles(rows) && tiles(inner)) && tiles(cols));
	V Cm = h.Allocate("C", {rows, cols}, TFType_Float);
	h.Dispatch(kernel, {Cm}, {A_in, B_in}, {rows, inner, cols}, {rows / h.Const(4), cols / h.Const(4)});
	h.Output(Cm);
	h.Finish();
}

static ProgramRegistrar reg_tiled_matmul_ir("tiled_matmul_ir", BuildTiledMatmulIr);

}  // namespace tfhost
