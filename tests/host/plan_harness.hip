// Host-only driver of the library's planning and validation code (cubework_amd/csrc/gemm_plan.hip with
// cw_runtime.hip's error text), built with the address and undefined-behaviour sanitizers on the host side
// (tests/test_host_sanitizers.py) and run on a machine without a GPU: no HIP call is made. It sweeps ragged,
// huge, zero and misaligned shapes through the same functions the entry points run and checks, for every plan,
// that the launches it describes stay inside the caller's buffers:
//   * a strip cut off for the small-tile kernel: head + tail cover the output exactly once, every shifted
//     pointer stays inside its operand, the strip fits one round of 128 x 128 tiles;
//   * the short extra step of a ragged reduction: starts at K - 32, its A part lies inside A, the scratch
//     copy of B's last rows fits the workspace that cw_gemm_workspace_bytes asked for;
//   * split k: slices divide K into multiples of 64, the partial sums fit the workspace;
//   * column sums: the slabs cover the rows exactly once and their partial rows fit cw_colsum_workspace_bytes'
//     promise of at most 512 (or ceil(M / 64)) rows.
// Prints "ok <checks> routes <how often each kernel route was planned>" and exits 0, or the first violated invariant and exits 1.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../cubework_amd/csrc/gemm_plan.h"

using namespace cw;

namespace {

long g_checked = 0;
long g_routes[6] = {0, 0, 0, 0, 0, 0};

#define REQUIRE(cond, ...)                                    \
    do {                                                      \
        if (!(cond)) {                                        \
            fprintf(stderr, "violated: %s | ", #cond);       \
            fprintf(stderr, __VA_ARGS__);                     \
            fprintf(stderr, "\n");                            \
            exit(1);                                          \
        }                                                     \
    } while (0)

struct Extent {
    const char* base;
    int64_t bytes;
};

bool inside(const void* p, int64_t need_bytes, const Extent& e) {
    const char* c = reinterpret_cast<const char*>(p);
    return c >= e.base && c + need_bytes <= e.base + e.bytes;
}

// Operands live in one fake address range per tensor (never dereferenced): the checks are on the arithmetic.
struct Problem {
    int layout;
    int64_t M, N, K, lda, ldb, ldc;
    int n_steps, n_addends;
    bool with_bias, with_preact, with_ws;
    int misalign;  // bytes added to A's base (0 = aligned)
};

int64_t a_rows(const Problem& p) { return p.layout == CW_TN ? p.K : p.M; }
int64_t a_cols(const Problem& p) { return p.layout == CW_TN ? p.M : p.K; }
int64_t b_rows(const Problem& p) { return p.layout == CW_NT ? p.N : p.K; }
int64_t b_cols(const Problem& p) { return p.layout == CW_NT ? p.K : p.N; }

void check_launch_extents(const GemmArgs& g, int layout, const Problem& p, const Extent (&A)[CW_MAX_KSTEPS],
                          const Extent (&B)[CW_MAX_KSTEPS], const Extent& C, const Extent& P, const Extent& bias,
                          const Extent (&add)[CW_MAX_ADDENDS], const char* what) {
    // the bytes a launch with these arguments touches: whole rows of its M x N output, its operands' used rows
    const int64_t ar = layout == CW_TN ? g.K : g.M, ac = layout == CW_TN ? g.M : g.K;
    const int64_t br = layout == CW_NT ? g.N : g.K, bc = layout == CW_NT ? g.K : g.N;
    REQUIRE(g.M > 0 && g.N > 0 && g.K >= 0, "%s: M=%d N=%d K=%d", what, g.M, g.N, g.K);
    for (int i = 0; i < g.n_steps; ++i) {
        REQUIRE(inside(g.A[i], ((ar - 1) * g.lda + ac) * 2, A[i]), "%s: A[%d] leaves its operand (M=%lld N=%lld K=%lld layout %d)", what,
                i, (long long)p.M, (long long)p.N, (long long)p.K, layout);
        REQUIRE(inside(g.B[i], ((br - 1) * g.ldb + bc) * 2, B[i]), "%s: B[%d] leaves its operand (M=%lld N=%lld K=%lld layout %d)", what,
                i, (long long)p.M, (long long)p.N, (long long)p.K, layout);
    }
    REQUIRE(inside(g.C, ((int64_t)(g.M - 1) * g.ldc + g.N) * 2, C), "%s: C leaves the output", what);
    if (g.preact != nullptr) REQUIRE(inside(g.preact, ((int64_t)(g.M - 1) * g.ldp + g.N) * 2, P), "%s: preact leaves its buffer", what);
    if (g.bias != nullptr) REQUIRE(inside(g.bias, (int64_t)g.N * 2, bias), "%s: bias leaves its vector", what);
    for (int j = 0; j < g.n_addends; ++j)
        REQUIRE(inside(g.addend[j], ((int64_t)(g.M - 1) * g.ldadd + g.N) * 2, add[j]), "%s: addend %d leaves its buffer", what, j);
}

void run_problem(const Problem& p) {
    // fake, well separated address ranges (1 TiB apart), 256-byte aligned
    auto range = [](int idx, int64_t bytes, int off) { return Extent{reinterpret_cast<const char*>(((int64_t)(idx + 1) << 40) + off), bytes}; };
    Extent A[CW_MAX_KSTEPS] = {}, B[CW_MAX_KSTEPS] = {}, add[CW_MAX_ADDENDS] = {};
    const void* a_tab[CW_MAX_KSTEPS] = {};
    const void* b_tab[CW_MAX_KSTEPS] = {};
    const void* add_tab[CW_MAX_ADDENDS] = {};
    for (int i = 0; i < p.n_steps && i < CW_MAX_KSTEPS; ++i) {
        A[i] = range(i, ((a_rows(p) - 1) * p.lda + a_cols(p)) * 2, p.misalign);
        B[i] = range(16 + i, ((b_rows(p) - 1) * p.ldb + b_cols(p)) * 2, 0);
        a_tab[i] = A[i].base;
        b_tab[i] = B[i].base;
    }
    const Extent C = range(40, ((p.M - 1) * p.ldc + p.N) * 2, 0), P = range(41, ((p.M - 1) * p.ldc + p.N) * 2, 0);
    const Extent bias = range(42, p.N * 2, 0);
    for (int j = 0; j < p.n_addends && j < CW_MAX_ADDENDS; ++j) {
        add[j] = range(48 + j, ((p.M - 1) * p.ldc + p.N) * 2, 0);
        add_tab[j] = add[j].base;
    }
    const int64_t ws_bytes = p.with_ws ? gemm_workspace_bytes(p.layout, p.M, p.N, p.K, p.n_steps, CW_BF16) : 0;
    REQUIRE(ws_bytes >= 0, "negative workspace size");
    const Extent W = range(60, ws_bytes, 0);
    GemmArgs args;
    bool nothing = false;
    const int rc = gemm_prepare_args(p.layout, p.M, p.N, p.K, p.n_steps, a_tab, p.lda, b_tab, p.ldb, p.with_bias ? bias.base : nullptr,
                                     p.with_bias ? CW_EPI_BIAS : CW_EPI_NONE, const_cast<char*>(C.base), p.ldc,
                                     p.with_preact ? const_cast<char*>(P.base) : nullptr, p.ldc, add_tab, p.n_addends, p.ldc,
                                     ws_bytes > 0 ? const_cast<char*>(W.base) : nullptr, ws_bytes, CW_BF16, &args, &nothing);
    ++g_checked;
    if (rc != CW_OK || nothing) return;  // refused (with a message) or empty: nothing is launched
    if (args.n_steps == 0) return;       // epilogue only
    for (int dma = 0; dma < 2; ++dma)
        for (int strip = 0; strip < 2; ++strip) {
            const GemmPlan plan = gemm_half_plan(args, p.layout, dma != 0, strip != 0);
            ++g_checked;
            REQUIRE(plan.route >= kRouteSmallRing && plan.route <= kRouteStaged, "route %d", plan.route);
            ++g_routes[plan.route];
            if (!dma) REQUIRE(plan.route == kRouteStaged, "CW_GEMM_IMPL=staged must reach the staged kernel, got route %d", plan.route);
            check_launch_extents(plan.head, p.layout, p, A, B, C, P, bias, add, "head");
            switch (plan.route) {
                case kRouteSmallRing:
                    REQUIRE(args.M >= 128 && args.N >= 128 && args.K % 64 == 0 && args.n_steps <= kRingMaxSteps, "small ring preconditions");
                    break;
                case kRouteRing:
                    REQUIRE(args.M >= 256 && args.N >= 256 && args.K % 32 == 0 && args.n_steps <= kRingMaxSteps && args.N % 8 == 0, "ring preconditions");
                    break;
                case kRouteRingThenSmall: {
                    const GemmArgs &h = plan.head, &t = plan.tail;
                    check_launch_extents(t, p.layout, p, A, B, C, P, bias, add, "tail");
                    REQUIRE((h.M == args.M && h.N + t.N == args.N && t.M == args.M) || (h.N == args.N && h.M + t.M == args.M && t.N == args.N),
                            "head %dx%d + tail %dx%d do not tile %dx%d", h.M, h.N, t.M, t.N, args.M, args.N);
                    REQUIRE(h.M % 256 == 0 || h.M == args.M, "head rows");
                    REQUIRE(h.N % 256 == 0 || h.N == args.N, "head columns");
                    REQUIRE(((int64_t)(t.M + 127) / 128) * ((t.N + 127) / 128) <= 256, "the strip is more than one round of small tiles");
                    REQUIRE(t.M >= 128 && t.N >= 128 && h.M >= 256 && h.N >= 256, "strip or head below one tile");
                    // the strip's output begins exactly where the head's ends
                    const char* c_end = reinterpret_cast<const char*>(h.C) + (h.N < args.N ? (int64_t)h.N * 2 : (int64_t)h.M * h.ldc * 2);
                    REQUIRE(reinterpret_cast<const char*>(t.C) == c_end, "the strip's output does not continue the head's");
                    break;
                }
                case kRouteRingKTail: {
                    const int kr = args.K % 32;
                    REQUIRE(kr != 0 && plan.head.K == args.K - kr && plan.head.K >= 32 && plan.ktail_zero_rows == 32 - kr, "k tail split");
                    REQUIRE(args.n_steps == 1 && p.layout != CW_NT, "k tail route");
                    const int64_t need = p.layout == CW_TN ? (31 * args.lda + args.M) * 2 : ((int64_t)(args.M - 1) * args.lda + 32) * 2;
                    REQUIRE(inside(plan.ktail_a, need, A[0]), "the extra step's A part leaves A");
                    REQUIRE(32 * args.ldb * 2 <= args.workspace_bytes, "the copy of B's last rows does not fit the workspace");
                    break;
                }
                case kRouteSplitK:
                    REQUIRE(plan.slices >= 2 && plan.slices <= 8 && args.K % (64 * plan.slices) == 0, "slices %d of K=%d", plan.slices, args.K);
                    REQUIRE((int64_t)plan.slices * args.M * args.N * 4 <= args.workspace_bytes, "partial sums exceed the workspace");
                    REQUIRE((int64_t)(args.M / 256) * (args.N / 256) * plan.slices <= 256 && args.M % 256 == 0 && args.N % 256 == 0, "split grid");
                    break;
                default: break;
            }
        }
}

void sweep_gemm() {
    const int64_t dims[] = {0, 1, 7, 8, 127, 128, 129, 255, 256, 264, 2040, 2048, 2056, 4096, 4352, 8192, 8704, 12568, 16384, 50272, 1 << 20};
    const int64_t ks[] = {0, 1, 8, 24, 32, 56, 64, 88, 2048, 2072, 4096, 8192, 12568, 16384};
    for (int layout = 0; layout < 3; ++layout)
        for (int64_t M : dims)
            for (int64_t N : dims)
                for (int64_t K : ks) {
                    if ((double)M * N > 4e11 || (double)M * K > 4e11 || (double)N * K > 4e11) continue;  // keep extents in int64
                    for (int variant = 0; variant < 6; ++variant) {
                        Problem p = {};
                        p.layout = layout;
                        p.M = M;
                        p.N = N;
                        p.K = K;
                        const int64_t pad = (variant == 1) ? 8 : (variant == 2 ? 3 : 0);
                        p.lda = (layout == CW_TN ? M : K) + pad;
                        p.ldb = (layout == CW_NT ? K : N) + pad;
                        p.ldc = N + pad;
                        p.n_steps = variant == 3 ? 4 : (variant == 4 ? 7 : (variant == 5 ? 2 : 1));
                        p.n_addends = variant == 4 ? 3 : (variant == 5 ? 2 : 0);
                        p.with_bias = variant != 0;
                        p.with_preact = variant == 5;
                        p.with_ws = variant != 2;
                        p.misalign = variant == 2 ? 2 : 0;
                        if (p.lda < 1) p.lda = 1;
                        if (p.ldb < 1) p.ldb = 1;
                        if (p.ldc < 1) p.ldc = 1;
                        run_problem(p);
                    }
                }
}

void check_refusals() {
    GemmArgs args;
    bool nothing = false;
    const void* tab[1] = {reinterpret_cast<const void*>(256)};
    void* c = reinterpret_cast<void*>(512);
    auto call = [&](int layout, int64_t M, int64_t N, int64_t K, int steps, const void* const* a, int64_t lda, const void* const* b,
                    int64_t ldb, void* C, int64_t ldc, int epi, int dt, int nadd) {
        return gemm_prepare_args(layout, M, N, K, steps, a, lda, b, ldb, nullptr, epi, C, ldc, nullptr, 0, nullptr, nadd, 0, nullptr, 0, dt,
                                 &args, &nothing);
    };
    REQUIRE(call(9, 8, 8, 8, 1, tab, 8, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "bad layout accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 8, tab, 8, c, 8, 9, 0, 0) == CW_ERR_INVALID, "bad epilogue accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 8, tab, 8, c, 8, 0, 7, 0) == CW_ERR_INVALID, "bad dtype accepted");
    REQUIRE(call(0, -1, 8, 8, 1, tab, 8, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "negative M accepted");
    REQUIRE(call(0, (int64_t)1 << 31, 8, 8, 1, tab, 8, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "M beyond int32 accepted");
    REQUIRE(call(0, 8, 8, 8, 99, tab, 8, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "99 steps accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 8, tab, 8, c, 8, 0, 0, 99) == CW_ERR_INVALID, "99 addends accepted");
    REQUIRE(call(0, 8, 8, 8, 1, nullptr, 8, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "NULL operand table accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 7, tab, 8, c, 8, 0, 0, 0) == CW_ERR_INVALID, "lda < K accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 8, tab, 8, nullptr, 8, 0, 0, 0) == CW_ERR_INVALID, "NULL C accepted");
    REQUIRE(call(0, 8, 8, 8, 1, tab, 8, tab, 8, c, 7, 0, 0, 0) == CW_ERR_INVALID, "ldc < N accepted");
    REQUIRE(call(0, 0, 8, 8, 1, tab, 8, tab, 8, nullptr, 8, 0, 0, 0) == CW_OK && nothing, "empty output must be a no-op");
    REQUIRE(gemm_workspace_bytes(CW_TN, 2048, 2048, 8192, 2, CW_BF16) == (int64_t)4 * 2048 * 2048 * 4, "split-k scratch of the weight gradient");
    REQUIRE(gemm_workspace_bytes(CW_TN, 2048, 2048, 8192, 2, CW_F32) == 0, "fp32 asks for no scratch");
    REQUIRE(gemm_workspace_bytes(CW_NN, -5, 2048, 8192, 2, CW_BF16) == 0 && gemm_workspace_bytes(7, 8, 8, 8, 1, CW_BF16) == 0, "bad arguments ask for no scratch");
    REQUIRE(gemm_workspace_bytes(CW_NN, (int64_t)1 << 40, (int64_t)1 << 40, 8192, 2, CW_BF16) == 0, "huge shapes ask for no scratch");
    g_checked += 16;
}

void sweep_colsum() {
    const int64_t ms[] = {1, 2, 15, 16, 17, 63, 64, 65, 300, 4095, 4096, 8192, 16384, 1 << 20, (int64_t)1 << 31};
    const int64_t ns[] = {1, 7, 8, 64, 512, 520, 2048, 8192, 8201, 50272, 1 << 20};
    for (int64_t M : ms)
        for (int64_t N : ns)
            for (int V : {4, 8})
                for (int vec = 0; vec < 2; ++vec) {
                    int64_t slabs = -1, rows = -1;
                    colsum_plan(M, N, V, vec != 0, slabs, rows);
                    ++g_checked;
                    REQUIRE(slabs >= 1 && rows >= 1, "colsum_plan(%lld, %lld): slabs %lld rows %lld", (long long)M, (long long)N, (long long)slabs, (long long)rows);
                    REQUIRE((slabs - 1) * rows < M && slabs * rows >= M, "slabs do not cover the rows exactly once (M=%lld N=%lld)", (long long)M, (long long)N);
                    if (vec) REQUIRE(slabs <= kColMaxSlabs, "more partial rows than the workspace bound");
                    else REQUIRE(slabs == (M + kColGenericSlabRows - 1) / kColGenericSlabRows, "generic slabs");
                }
}

}  // namespace

int main() {
    check_refusals();
    sweep_colsum();
    sweep_gemm();
    printf("ok %ld routes small_ring=%ld ring=%ld ring_then_small=%ld ring_ktail=%ld split_k=%ld staged=%ld\n", g_checked, g_routes[0],
           g_routes[1], g_routes[2], g_routes[3], g_routes[4], g_routes[5]);
    return 0;
}
