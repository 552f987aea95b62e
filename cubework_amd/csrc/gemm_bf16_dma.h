// SUMMA block GEMM for gfx950, large tile-aligned problems: 256x256 tile of C
// per 256-thread block, operands streamed global -> LDS by the load unit itself
// (global_load_lds_dwordx4: no staging registers, no LDS write instructions, no
// transposition ALU work), fragments read with ds_read_b128 (operand stored with
// k contiguous) or ds_read_b64_tr_b16 (operand stored with k as the slow index:
// the LDS read transposes 4x4 blocks across 16 lanes), fp32 accumulation in
// v_mfma_f32_32x32x16_bf16, the same epilogue as the register-staged kernel.
//
// LDS image of one stage (k extent 64), per operand 32 KB:
//   k-contiguous operand  : [256 rows][64 k], 128 B per row, 16-byte chunk c of
//     row r stored at chunk position c ^ ((r >> 1) & 7): the 16 rows a
//     half-wavefront reads at one k offset fall in 16 different bank groups.
//   k-slow operand        : [64 k][256 rows], 512 B per k row, chunk c of k row k
//     stored at position c ^ ((k & 3) << 2): the four k rows one transposing
//     read touches fall in four different 64-byte bank windows.
// A load instruction writes 1 KB of LDS linearly (lane l -> bytes [16l, 16l+16)),
// so the swizzle is applied on the global side: lane l fetches the chunk that
// belongs at its LDS position.
#pragma once

#include "gemm_bf16_kernel.h"

namespace cw {
namespace gemm_dma {

using gemm_bf16::bf16x8_t;
using gemm_bf16::f32x16_t;

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));

constexpr int kTile = 256;               // BM = BN
constexpr int kBK = 64;
constexpr int kThreads = 256;
constexpr int kOperBytes = kTile * kBK * 2;   // 32768
constexpr int kStageBytes = 2 * kOperBytes;   // 65536
constexpr int kStages = 2;

typedef __attribute__((address_space(3))) char lds_char;

// One LDS-DMA load: lane l copies 16 bytes from gbase + voff to LDS address
// lds_addr + 16*l. gbase and lds_addr are wavefront-uniform. Issued through
// inline asm on purpose: the compiler cannot tell the transposing LDS reads
// apart from these LDS writes and would wait for every outstanding load before
// each of them; the kernel waits on the load counter itself (dma_wait_all)
// before the barrier that publishes a stage.
__device__ __forceinline__ void dma16(const char* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(gbase)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Per-thread byte offsets of the chunk a lane fetches, for even / odd load
// instructions of its wavefront (the swizzle term alternates with the
// instruction index). row0: first row (m0 or n0) of the tile in the operand.
template <bool TRANS>
__device__ __forceinline__ void dma_lane_offsets(int lane, int64_t ld, int row0, uint32_t& even, uint32_t& odd) {
    if constexpr (!TRANS) {
        // instruction = 8 rows x 128 B; lane -> row lane/8, LDS chunk position lane%8
        const int r = lane >> 3, cpos = lane & 7;
        const int c_even = cpos ^ (lane >> 4);        // swizzle ((row>>1)&7) = (lane>>4) + 4*(it&1)
        const int c_odd = c_even ^ 4;
        even = (uint32_t)((((int64_t)(row0 + r)) * ld + c_even * 8) * 2);
        odd = (uint32_t)((((int64_t)(row0 + r)) * ld + c_odd * 8) * 2);
    } else {
        // instruction = 2 k rows x 512 B; lane -> k row lane/32, LDS chunk position lane%32
        const int kr = lane >> 5, cpos = lane & 31;
        const int c_even = cpos ^ (kr << 2);          // k & 3 = 2*(it&1) + lane/32
        const int c_odd = cpos ^ ((2 + kr) << 2);
        even = (uint32_t)((((int64_t)kr) * ld + row0 + c_even * 8) * 2);
        odd = (uint32_t)((((int64_t)kr) * ld + row0 + c_odd * 8) * 2);
    }
}

// Issue this wavefront's 8 load instructions of one operand tile.
// gbase: operand base of the current k-step (uniform); k0: first k of the tile.
template <bool TRANS>
__device__ __forceinline__ void dma_tile(const char* gbase, int64_t ld_bytes, int k0, uint32_t voff_even,
                                         uint32_t voff_odd, uint32_t lds_oper, int wave) {
    gemm_bf16::static_for<8>([&](auto it) {
        constexpr int I = it.value;
        const uint32_t voff = (I & 1) ? voff_odd : voff_even;
        if constexpr (!TRANS) {
            const int row = wave * 64 + I * 8;  // rows [row, row+8)
            const char* p = gbase + ((int64_t)row * ld_bytes + (int64_t)k0 * 2);
            dma16(p, voff, lds_oper + row * 128);
        } else {
            const int k = wave * 16 + I * 2;    // k rows [k, k+2)
            const char* p = gbase + (int64_t)(k0 + k) * ld_bytes;
            dma16(p, voff, lds_oper + k * 512);
        }
    });
}

// Fragment addressing of one operand for a wavefront whose 128 rows start at
// row `wrow` of the tile. frag(t, ks): 8 k values (k = ks*16 + 8*(lane/32) + 0..7)
// of row wrow + t*32 + lane%32.
template <bool TRANS>
struct FragReader {
    uint32_t off[4];  // !TRANS: per ks;  TRANS: per t
    __device__ __forceinline__ void init(int lane, int wrow) {
        if constexpr (!TRANS) {
            const int r = lane & 31, g = lane >> 5;
            const int swz = (r >> 1) & 7;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) off[ks] = (uint32_t)((wrow + r) * 128 + (((2 * ks + g) ^ swz) << 4));
        } else {
            const int i = lane & 15, grp = lane >> 4;
            const int g = grp >> 1, kk = (i >> 2) & 3;
            const int lane_const = (8 * g + (i >> 2)) * 512 + (((wrow >> 3) + 2 * (grp & 1) + ((i & 3) >> 1)) << 4) + 8 * (i & 1);
#pragma unroll
            for (int t = 0; t < 4; ++t) off[t] = (uint32_t)(lane_const + 64 * (t ^ kk));
        }
    }
    template <int T, int KS>
    __device__ __forceinline__ bf16x8_t read(lds_char* oper) const {
        if constexpr (!TRANS) {
            return *(__attribute__((address_space(3))) const bf16x8_t*)(oper + off[KS] + T * 32 * 128);
        } else {
            lds_char* p = oper + off[T] + KS * 16 * 512;
            const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
            const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 4 * 512));
            const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(bf16x8_t, v);
        }
    }
};

template <bool TRANS_A, bool TRANS_B, int EPI>
__global__ __launch_bounds__(kThreads) void gemm_bf16_dma_kernel(const GemmArgs args) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    lds_char* lds_base = (lds_char*)lds;
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)lds_base;  // LDS byte address of the dynamic segment

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    const int M = args.M, N = args.N, K = args.K;
    const int tiles_m = M / kTile, tiles_n = N / kTile;
    const int total = tiles_m * tiles_n;
    int tile;
    {
        // ids pid, pid+8, ... run on one XCD: give each XCD a contiguous range of tiles
        const int pid = blockIdx.x;
        const int per_xcd = (total + 7) / 8;
        tile = (pid & 7) * per_xcd + (pid >> 3);
        if (tile >= total) return;
    }
    constexpr int GROUP_M = 8;
    const int group = tile / (GROUP_M * tiles_n);
    const int first_m = group * GROUP_M;
    const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = tile - group * GROUP_M * tiles_n;
    const int m0 = (first_m + in_group % gsz) * kTile;
    const int n0 = (in_group / gsz) * kTile;

    const int kt_per_step = K / kBK;
    const int KT = kt_per_step * args.n_steps;

    uint32_t a_even, a_odd, b_even, b_odd;
    dma_lane_offsets<TRANS_A>(lane, args.lda, m0, a_even, a_odd);
    dma_lane_offsets<TRANS_B>(lane, args.ldb, n0, b_even, b_odd);
    const int64_t lda_bytes = args.lda * 2, ldb_bytes = args.ldb * 2;

    FragReader<TRANS_A> fa;
    FragReader<TRANS_B> fb;
    fa.init(lane, wm * 128);
    fb.init(lane, wn * 128);

    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto issue_tile = [&](int kt, int stage) {
        const int step = kt / kt_per_step;
        const int k0 = (kt - step * kt_per_step) * kBK;
        const uint32_t st = lds_addr0 + stage * kStageBytes;
        dma_tile<TRANS_A>(reinterpret_cast<const char*>(args.A[step]), lda_bytes, k0, a_even, a_odd, st, wave);
        dma_tile<TRANS_B>(reinterpret_cast<const char*>(args.B[step]), ldb_bytes, k0, b_even, b_odd, st + kOperBytes, wave);
    };

    if (KT > 0) issue_tile(0, 0);

    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        // own loads of tile kt have landed; after the barrier everybody's have,
        // and every wave is past its reads of the other stage
        dma_wait_all();
        __syncthreads();
        if (kt + 1 < KT) issue_tile(kt + 1, cur ^ 1);
        lds_char* sa = lds_base + cur * kStageBytes;
        lds_char* sb = sa + kOperBytes;

        bf16x8_t af[2][4], bfr[2][4];
        gemm_bf16::static_for<4>([&](auto t) {
            af[0][t.value] = fa.template read<t.value, 0>(sa);
            bfr[0][t.value] = fb.template read<t.value, 0>(sb);
        });
        gemm_bf16::static_for<4>([&](auto ks) {
            constexpr int KS = ks.value;
            if constexpr (KS + 1 < 4) {
                gemm_bf16::static_for<4>([&](auto t) {
                    af[(KS + 1) & 1][t.value] = fa.template read<t.value, KS + 1>(sa);
                    bfr[(KS + 1) & 1][t.value] = fb.template read<t.value, KS + 1>(sb);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[KS & 1][j], af[KS & 1][i], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
    }
    __syncthreads();  // all operand reads done: the stages become the C tile
    gemm_bf16::gemm_epilogue<kTile, kTile, 4, 4, EPI>(acc, args, lds, m0, n0, wm, wn, lane, tid);
}

constexpr size_t lds_bytes_dma() {
    const size_t stages = (size_t)kStages * kStageBytes;
    const size_t ctile = (size_t)kTile * (kTile + 4) * sizeof(uint16_t);
    return stages > ctile ? stages : ctile;
}

template <bool TA, bool TB, int EPI>
int launch_dma_cfg(const GemmArgs& args, hipStream_t s) {
    auto kern = gemm_bf16_dma_kernel<TA, TB, EPI>;
    constexpr size_t lds = lds_bytes_dma();
    static_assert(lds <= 160 * 1024, "LDS image does not fit the CU");
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail(CW_ERR_LAUNCH, "hipFuncSetAttribute(gemm_bf16_dma): %s", hipGetErrorString(e));
    const int tiles = (args.M / kTile) * (args.N / kTile);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, s, args);
    return check_launch("gemm_bf16_dma_kernel");
}

template <bool TA, bool TB>
int launch_dma(const GemmArgs& args, int epilogue, hipStream_t s) {
    switch (epilogue) {
        case CW_EPI_NONE: return launch_dma_cfg<TA, TB, CW_EPI_NONE>(args, s);
        case CW_EPI_BIAS: return launch_dma_cfg<TA, TB, CW_EPI_BIAS>(args, s);
        case CW_EPI_BIAS_GELU_TANH: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_GELU_TANH>(args, s);
        case CW_EPI_BIAS_GELU_ERF: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_GELU_ERF>(args, s);
        case CW_EPI_BIAS_RELU: return launch_dma_cfg<TA, TB, CW_EPI_BIAS_RELU>(args, s);
        default: return fail(CW_ERR_INVALID, "cw_gemm_ksteps: bad epilogue %d", epilogue);
    }
}

}  // namespace gemm_dma
}  // namespace cw
