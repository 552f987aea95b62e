// Host-side planning of the block GEMM and of the column sums: argument validation, which kernel takes a
// shape, how a product is cut into launches (a strip of tile rows / columns for the small-tile kernel, the
// short extra step that finishes a ragged reduction, k slices) and how much scratch that needs. Pure integer
// and pointer arithmetic with no HIP call, so that the same functions the entry points run can be driven on a
// machine without a GPU under the address and undefined-behaviour sanitizers (tests/host/plan_harness.hip):
// this is the arithmetic where an off-by-one becomes an out-of-bounds access on the device.
#pragma once

#include "gemm.h"

namespace cw {

// Checks the arguments of cw_gemm_ksteps(_ws) (the reference's assertion on mismatched operand shapes,
// cubework/module/parallel_2d/_operation.py:30, and what a C ABI has to add: null pointers, leading
// dimensions, counts) and fills the kernels' argument block with its alignment flags. Returns CW_OK, or an
// error code with the thread's error text set. *nothing_to_do is set when M or N is zero (CW_OK, no launch).
int gemm_prepare_args(int layout, int64_t M, int64_t N, int64_t K, int n_steps, const void* const* A_steps, int64_t lda,
                      const void* const* B_steps, int64_t ldb, const void* bias, int epilogue, void* C, int64_t ldc,
                      void* preact, int64_t ldp, const void* const* addends, int n_addends, int64_t ldadd, void* workspace,
                      int64_t workspace_bytes, int io_dtype, GemmArgs* out, bool* nothing_to_do);

// Scratch that enables the split-k launch or the ragged-reduction step for a 16-bit product (0: neither).
int64_t gemm_workspace_bytes(int layout, int64_t M, int64_t N, int64_t K, int n_steps, int io_dtype);

enum GemmRoute {
    kRouteSmallRing = 0,      // 128 x 128 tiles, ring of LDS stages filled by the load unit
    kRouteRing = 1,           // 256 x 256 tiles, the same ring
    kRouteRingThenSmall = 2,  // whole rounds of 256 x 256 tiles (head), the mostly empty last round as 128 x 128 tiles (tail)
    kRouteRingKTail = 3,      // ring + one short step over k in [K-32, K) for K % 32 != 0 (B stored [K, N])
    kRouteSplitK = 4,         // ring over k slices into fp32 partials, then the reduce / epilogue launch
    kRouteStaged = 5,         // register-staged kernel (ragged, unaligned, > 4 k-steps)
};

struct GemmPlan {
    int route;
    GemmArgs head;            // the launch of every route (kRouteRingKTail: K already shortened to a multiple of 32)
    GemmArgs tail;            // kRouteRingThenSmall only: the strip
    int slices;               // kRouteSplitK
    bool big, exact;          // kRouteStaged: 256 x 256 tiles / unguarded instantiation
    const void* ktail_a;      // kRouteRingKTail: A's part of the extra step (inside A[0])
    int ktail_zero_rows;      // kRouteRingKTail: leading rows of the copied 32 rows of B that must be zero
};

// dma_enabled / strip_enabled: the two CW_GEMM_IMPL switches (staged / onelaunch) as the caller read them.
GemmPlan gemm_half_plan(const GemmArgs& args, int layout, bool dma_enabled, bool strip_enabled);

// Row slabs of the column-sum kernels for an [M, N] operand with V elements per 16 bytes: one partial row of N
// sums per slab (vec: the vector kernel takes the shape; else the element-wise kernel).
void colsum_plan(int64_t M, int64_t N, int V, bool vec, int64_t& slabs, int64_t& rows_per_slab);
constexpr int kColWaves = 4;                 // wavefronts per block of the vector kernel, each on its own rows
constexpr int kColUnroll = 4;                // rows in flight per wavefront
constexpr int64_t kColBlocks = 1024;         // blocks aimed at (4 resident per compute unit)
constexpr int64_t kColGenericSlabRows = 64;  // rows per slab of the element-wise kernel
constexpr int64_t kColMaxSlabs = 512;        // the bound cw_colsum_workspace_bytes promises

}  // namespace cw
