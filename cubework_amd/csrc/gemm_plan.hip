// Host-side planning of the block GEMM and the column sums (declared in gemm_plan.h): no HIP call, no kernel.
#include <cstring>

#include "gemm_plan.h"
#include "gemm_bf16_kernel.h"

namespace cw {

int gemm_bf16_split_slices(int64_t M, int64_t N, int64_t K, int n_steps) {
    if (M <= 0 || N <= 0 || K <= 0 || n_steps <= 0 || n_steps > kRingMaxSteps) return 1;
    if ((M % 256) != 0 || (N % 256) != 0 || (K % 64) != 0) return 1;
    const int64_t tiles = (M / 256) * (N / 256);
    if (tiles >= 128 || K * n_steps < 2048) return 1;  // enough tiles already, or a short reduction
    int slices = 8;
    while (slices > 1 && (tiles * slices > 256 || (K % (64 * slices)) != 0 || K / slices < 256)) slices >>= 1;
    return slices;
}

int64_t gemm_bf16_ktail_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps) {
    if (layout == CW_NT || n_steps != 1 || K < 64 || (K % 32) == 0 || (K % 8) != 0) return 0;
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    if (tiles < 128 || M < 256 || N < 256 || (N % 8) != 0) return 0;
    return 32 * N * (int64_t)sizeof(uint16_t);
}

int64_t gemm_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps, int io_dtype) {
    if (layout != CW_NN && layout != CW_NT && layout != CW_TN) return 0;
    if (io_dtype != CW_BF16 && io_dtype != CW_F16) return 0;  // the fp32 GEMM is not split
    if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
    const int slices = gemm_bf16_split_slices(M, N, K, n_steps);
    if (slices > 1) {
        // shapes the 128 x 128 ring kernel takes in preference to the split (gemm_half_plan) need none
        const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
        if (tiles128 >= 192 && K * n_steps < 12288) return 0;
        return (int64_t)slices * M * N * (int64_t)sizeof(float);
    }
    return gemm_bf16_ktail_workspace_bytes(layout, M, N, K, n_steps);
}

int gemm_prepare_args(int layout, int64_t M, int64_t N, int64_t K, int n_steps, const void* const* A_steps, int64_t lda,
                      const void* const* B_steps, int64_t ldb, const void* bias, int epilogue, void* C, int64_t ldc,
                      void* preact, int64_t ldp, const void* const* addends, int n_addends, int64_t ldadd, void* workspace,
                      int64_t workspace_bytes, int io_dtype, GemmArgs* out, bool* nothing_to_do) {
    *nothing_to_do = false;
    if (layout != CW_NN && layout != CW_NT && layout != CW_TN)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad layout %d", layout);
    if (epilogue < CW_EPI_NONE || epilogue > CW_EPI_BIAS_RELU)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    if (io_dtype != CW_BF16 && io_dtype != CW_F32 && io_dtype != CW_F16)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad io_dtype %d", io_dtype);
    if (M < 0 || N < 0 || K < 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                    (long long)K);
    if (n_steps < 0 || n_steps > CW_MAX_KSTEPS)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: n_steps=%d outside [0, %d]", n_steps, CW_MAX_KSTEPS);
    if (n_addends < 0 || n_addends > CW_MAX_ADDENDS)
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: n_addends=%d outside [0, %d]", n_addends, CW_MAX_ADDENDS);
    if (M == 0 || N == 0) {
        *nothing_to_do = true;
        return CW_OK;
    }
    if (C == nullptr || ldc < N) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: C is NULL or ldc < N");
    if (preact != nullptr && ldp < N) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: ldp < N");
    if (K == 0) n_steps = 0;
    if (n_steps > 0) {
        if (A_steps == nullptr || B_steps == nullptr)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: operand pointer tables are NULL");
        const int64_t a_cols = (layout == CW_TN) ? M : K;  // contiguous extent of A's rows
        const int64_t b_cols = (layout == CW_NT) ? K : N;
        if (lda < a_cols || ldb < b_cols)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: leading dimension smaller than the row (lda=%lld ldb=%lld)",
                        (long long)lda, (long long)ldb);
    }
    if (n_addends > 0 && (addends == nullptr || ldadd < N))
        return fail(CW_ERR_INVALID, "cw_gemm_ksteps: addends table is NULL or ldadd < N");

    GemmArgs args;
    memset(&args, 0, sizeof(args));
    const int vec = (io_dtype == CW_F32) ? 4 : 8;        // elements per 16 bytes
    const uintptr_t out_mask = 15u;                      // outputs / addends move 16 bytes at a time
    const int out_vec = (io_dtype == CW_F32) ? 4 : 8;    // elements per 16 bytes
    args.vec_a = args.vec_b = 1;
    for (int i = 0; i < n_steps; ++i) {
        if (A_steps[i] == nullptr || B_steps[i] == nullptr)
            return fail(CW_ERR_INVALID, "cw_gemm_ksteps: operand pointer of step %d is NULL", i);
        args.A[i] = A_steps[i];
        args.B[i] = B_steps[i];
        if (!aligned16(A_steps[i])) args.vec_a = 0;
        if (!aligned16(B_steps[i])) args.vec_b = 0;
    }
    if (lda % vec != 0) args.vec_a = 0;
    if (ldb % vec != 0) args.vec_b = 0;
    args.vec_add = 1;
    for (int j = 0; j < n_addends; ++j) {
        if (addends[j] == nullptr) return fail(CW_ERR_INVALID, "cw_gemm_ksteps: addend %d is NULL", j);
        args.addend[j] = addends[j];
        if ((reinterpret_cast<uintptr_t>(addends[j]) & out_mask) != 0) args.vec_add = 0;
    }
    if (ldadd % out_vec != 0) args.vec_add = 0;
    args.bias = bias;
    args.vec_bias = (bias == nullptr || (reinterpret_cast<uintptr_t>(bias) & 7u) == 0) ? 1 : 0;
    args.C = C;
    args.vec_c = ((reinterpret_cast<uintptr_t>(C) & out_mask) == 0 && ldc % out_vec == 0) ? 1 : 0;
    args.preact = preact;
    args.vec_p = (preact == nullptr || ((reinterpret_cast<uintptr_t>(preact) & out_mask) == 0 && ldp % out_vec == 0)) ? 1 : 0;
    args.lda = lda;
    args.ldb = ldb;
    args.ldc = ldc;
    args.ldp = ldp;
    args.ldadd = ldadd;
    args.M = (int)M;
    args.N = (int)N;
    args.K = (int)K;
    args.n_steps = n_steps;
    args.n_addends = n_addends;
    args.workspace = workspace_bytes > 0 ? workspace : nullptr;
    args.workspace_bytes = workspace != nullptr ? workspace_bytes : 0;
    *out = args;
    return CW_OK;
}

GemmPlan gemm_half_plan(const GemmArgs& args, int layout, bool dma_enabled, bool strip_enabled) {
    GemmPlan plan;
    memset(&plan, 0, sizeof(plan));
    plan.head = args;
    plan.tail = args;
    plan.slices = 1;
    // the unguarded kernels address operands with 32-bit byte offsets
    const int64_t max_dim = args.M > args.N ? (args.M > args.K ? args.M : args.K) : (args.N > args.K ? args.N : args.K);
    const bool fits32 = (max_dim + 64) * (args.lda > args.ldb ? args.lda : args.ldb) * 2 < ((int64_t)1 << 32);
    const bool all_vec = fits32 && args.vec_a && args.vec_b && args.vec_c && (args.preact == nullptr || args.vec_p) &&
                         (args.bias == nullptr || args.vec_bias) && (args.n_addends == 0 || args.vec_add);
    const int64_t tiles256 = (int64_t)((args.M + 255) / 256) * ((args.N + 255) / 256);
    const bool big = tiles256 >= 128;
    const int tile = big ? 256 : 128;
    const bool exact = all_vec && (args.M % tile) == 0 && (args.N % tile) == 0 && (args.K % gemm_bf16::kBK) == 0;
    plan.big = big;
    plan.exact = exact;
    const bool ring_ok = args.n_steps > 0 && args.n_steps <= kRingMaxSteps && args.n_addends <= kRingMaxAddends && dma_enabled;
    // The LDS-DMA kernel takes M and N that are not tile multiples (its last tiles overlap their
    // neighbours): a vocabulary slice of 12568 columns is 50 tiles instead of 49.1. What it needs is one
    // full tile in each direction and 16-byte steps wherever a tile origin moves along a contiguous
    // dimension (N always: the output and a [K, N] operand; M for a [K, M] operand).
    const bool edges_ok = args.M >= 256 && args.N >= 256 && (args.N % 8) == 0 && (layout != CW_TN || (args.M % 8) == 0);
    // Fewer than 160 tiles of 256 x 256 (at 128 .. 159 of them the large tiles leave 40 % of the compute units
    // idle, and four times as many small tiles fill them): the ring kernel with 128 x 128 tiles, unless a long
    // reduction over few tiles is better served by splitting k (below; measured on 2048 x 2048 outputs: the
    // small tiles win up to a reduction length of 8192, the split from 16384).
    const int slices = gemm_bf16_split_slices(args.M, args.N, args.K, args.n_steps);
    const bool splits = slices > 1 && args.workspace != nullptr && aligned16(args.workspace) &&
                        args.workspace_bytes >= (int64_t)slices * args.M * args.N * (int64_t)sizeof(float);
    {
        const int64_t tiles128 = (int64_t)((args.M + 127) / 128) * ((args.N + 127) / 128);
        if (tiles256 < 160 && all_vec && ring_ok && args.M >= 128 && args.N >= 128 && (args.N % 8) == 0 &&
            (layout != CW_TN || (args.M % 8) == 0) && args.K >= 64 && (args.K % 64) == 0 &&
            args.lda < ((int64_t)1 << 23) && args.ldb < ((int64_t)1 << 23) &&
            ((tiles128 >= 192 && (int64_t)args.K * args.n_steps < 12288) || !splits)) {
            plan.route = kRouteSmallRing;
            return plan;
        }
    }
    if (big && all_vec && ring_ok && edges_ok && (args.K % gemm_bf16::kBK) == 0) {
        // A last round of 256 x 256 tiles that is mostly empty (a vocabulary slice as N: 8192 x 12568 is 32 x 50 =
        // 1600 tiles, 6.25 rounds of the 256 compute units): when the partial round is whole tile columns (or whole
        // tile rows), at most 3/8 of a round, and that strip is at most one round of 128 x 128 tiles, it goes to the
        // small-tile kernel as a second launch and the rest is whole rounds.
        const int64_t tiles_m = (args.M + 255) / 256, tiles_n = (args.N + 255) / 256;
        const int64_t last_round = (tiles_m * tiles_n) % 256;
        const bool small_ok = (args.K % 64) == 0 && args.lda < ((int64_t)1 << 23) && args.ldb < ((int64_t)1 << 23);
        if (tiles_m * tiles_n > 256 && last_round > 0 && last_round <= 96 && small_ok && strip_enabled) {
            auto shift = [&](const void* p, int64_t elems) -> const void* {
                return p == nullptr ? nullptr : reinterpret_cast<const uint16_t*>(p) + elems;
            };
            GemmArgs& head = plan.head;
            GemmArgs& tail = plan.tail;
            bool split = false;
            if (last_round % tiles_m == 0) {  // whole tile columns
                const int64_t n0 = (tiles_n - last_round / tiles_m) * 256, strip = args.N - n0;
                if (n0 >= 256 && strip >= 128 && ((args.M + 127) / 128) * ((strip + 127) / 128) <= 256) {
                    head.N = (int)n0;
                    tail.N = (int)strip;
                    for (int i = 0; i < args.n_steps; ++i) tail.B[i] = shift(args.B[i], layout == CW_NT ? n0 * args.ldb : n0);
                    for (int k = 0; k < args.n_addends; ++k) tail.addend[k] = shift(args.addend[k], n0);
                    tail.bias = shift(args.bias, n0);
                    tail.C = const_cast<void*>(shift(args.C, n0));
                    tail.preact = const_cast<void*>(shift(args.preact, n0));
                    split = true;
                }
            }
            if (!split && last_round % tiles_n == 0) {  // whole tile rows
                const int64_t m0 = (tiles_m - last_round / tiles_n) * 256, strip = args.M - m0;
                if (m0 >= 256 && strip >= 128 && ((strip + 127) / 128) * ((args.N + 127) / 128) <= 256) {
                    head.M = (int)m0;
                    tail.M = (int)strip;
                    for (int i = 0; i < args.n_steps; ++i) tail.A[i] = shift(args.A[i], layout == CW_TN ? m0 : m0 * args.lda);
                    for (int k = 0; k < args.n_addends; ++k) tail.addend[k] = shift(args.addend[k], m0 * args.ldadd);
                    tail.C = const_cast<void*>(shift(args.C, m0 * args.ldc));
                    tail.preact = const_cast<void*>(shift(args.preact, m0 * args.ldp));
                    split = true;
                }
            }
            if (split) {
                plan.route = kRouteRingThenSmall;
                return plan;
            }
        }
        plan.route = kRouteRing;
        return plan;
    }
    // A reduction length that is not a multiple of the k tile (a vocabulary slice as K: 12568 = 392 x 32 +
    // 24), with B stored [K, N]: the regular step covers the first K - K % 32 columns, one more step of 32
    // covers [K-32, K) with a copy of B's last 32 rows whose overlapping rows are zero. The copy (64 bytes
    // per column) lives in the caller's scratch and has B's row pitch, which the steps share.
    if (big && all_vec && ring_ok && edges_ok && layout != CW_NT && args.n_steps == 1 && args.K >= 64 &&
        (args.K % 32) != 0 && (args.K % 8) == 0 && args.workspace != nullptr && aligned16(args.workspace) &&
        args.workspace_bytes >= 32 * args.ldb * (int64_t)sizeof(uint16_t)) {
        const int kr = args.K % 32;
        // A's part of the step: columns (NN, A is [M, K]) or rows (TN, A is [K, M]) K-32 .. K-1, in place
        const uint16_t* a0 = reinterpret_cast<const uint16_t*>(args.A[0]);
        plan.ktail_a = layout == CW_TN ? a0 + (int64_t)(args.K - 32) * args.lda : a0 + (args.K - 32);
        plan.ktail_zero_rows = 32 - kr;
        plan.head.K = args.K - kr;
        plan.route = kRouteRingKTail;
        return plan;
    }
    if (splits && all_vec && args.n_addends <= kRingMaxAddends && dma_enabled) {
        plan.slices = slices;
        plan.route = kRouteSplitK;
        return plan;
    }
    plan.route = kRouteStaged;
    return plan;
}

void colsum_plan(int64_t M, int64_t N, int V, bool vec, int64_t& slabs, int64_t& rows_per_slab) {
    if (!vec) {
        rows_per_slab = kColGenericSlabRows;
        slabs = (M + rows_per_slab - 1) / rows_per_slab;
        return;
    }
    const int64_t coltiles = (N + 64 * V - 1) / (64 * V);
    slabs = kColBlocks / coltiles;
    const int64_t max_slabs = (M + kColWaves * kColUnroll - 1) / (kColWaves * kColUnroll);
    if (slabs > max_slabs) slabs = max_slabs;
    if (slabs > kColMaxSlabs) slabs = kColMaxSlabs;
    if (slabs < 1) slabs = 1;
    rows_per_slab = (M + slabs - 1) / slabs;
    slabs = (M + rows_per_slab - 1) / rows_per_slab;
}

}  // namespace cw
