// Pieces shared by the attention forward and backward kernels (gfx950; bf16, or fp16 with E = f16_t):
// LDS tile images of 64 columns (a head of 128 is two of them side by side),
// MFMA operand reads, tile loader.
#pragma once

#include <type_traits>

#include "cw_common.h"

namespace cw {
namespace attn {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) char lds_char;

constexpr int kHead = 64;                  // columns of one LDS image (a head of 128 is two images side by side)
constexpr int kTile = 64;                  // rows of a streamed tile
constexpr int kImage = kTile * kHead * 2;  // 8 KB: one LDS image of a tile
constexpr float kNegBig = -__builtin_huge_valf();

// A 64-row tile ([row][64 bf16], 128 bytes per row) is kept in LDS in one or
// both of two images:
//   row image       : 16-byte chunk c of row r at position c ^ ((r >> 1) & 7); read with ds_read_b128 as
//                     the MFMA operand "row = r0 + lane % 32, k = 8 values at 16 kb + 8 (lane / 32)";
//   transpose image : chunk c of row r inside 32-byte unit (c >> 1) ^ (r & 3); read with
//                     ds_read_b64_tr_b16 as the operand "row = column 32 dt + lane % 32 of the tile,
//                     k slots = tile rows r0 + 4 (lane / 32) + {0..3} and + 8 + {0..3}".
// Both read patterns are free of bank conflicts (SQ_LDS_BANK_CONFLICT = 0).
__device__ __forceinline__ int row_image_offset(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
__device__ __forceinline__ int tr_image_offset(int r, int c) { return r * 128 + ((((c >> 1) ^ (r & 3)) << 5) | ((c & 1) << 4)); }

// Per-lane byte offsets of the two read patterns, computed once. A read adds a
// compile-time row offset (a multiple of 16 rows, which leaves the swizzle
// terms unchanged) as the instruction's immediate.
struct ReadOffsets {
    int rows[4];  // [kb]
    int tr[2];    // [dt]
    __device__ __forceinline__ void init(int lane) {
        const int l32 = lane & 31, half = lane >> 5, grp = lane >> 4, i16 = lane & 15;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) rows[kb] = row_image_offset(l32, 2 * kb + half);
        const int ra = 4 * (grp >> 1) + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) tr[dt] = ra * 128 + (((2 * dt + (grp & 1)) ^ (ra & 3)) << 5) + 8 * (i16 & 3);
    }
};

template <int R0>
__device__ __forceinline__ bf16x8_t read_rows(lds_char* img, const ReadOffsets& ro, int kb) {
    static_assert(R0 % 16 == 0, "row offset must keep the swizzle");
    return *(__attribute__((address_space(3))) const bf16x8_t*)(img + ro.rows[kb] + R0 * 128);
}
template <int R0>
__device__ __forceinline__ bf16x8_t read_transposed(lds_char* img, const ReadOffsets& ro, int dt) {
    static_assert(R0 % 16 == 0, "row offset must keep the swizzle");
    lds_char* p = img + ro.tr[dt] + R0 * 128;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)p);
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p + 8 * 128));
    return __builtin_bit_cast(bf16x8_t, (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// Operands travel as 8 x 16 bits (bf16x8_t) whatever the element type E (bf16_t or f16_t); these are
// the places where the type matters.
template <typename E>
__device__ __forceinline__ f32x16_t mfma16(bf16x8_t a, bf16x8_t b, f32x16_t acc) {
    if constexpr (std::is_same<E, f16_t>::value)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
// B operand from 8 consecutive accumulator elements (k slot j <-> element 8 blk + j), rounded to E.
template <typename E>
__device__ __forceinline__ bf16x8_t pack_slots(const float (&x)[16], int blk) {
    if constexpr (std::is_same<E, f16_t>::value) {
        f16x8_t r;
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = (_Float16)x[8 * blk + j];
        return __builtin_bit_cast(bf16x8_t, r);
    } else {
        bf16x8_t r;
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = (__bf16)x[8 * blk + j];
        return r;
    }
}
// Sum of the 8 values of an operand, in fp32 (v_dot2 with ones).
template <typename E>
__device__ __forceinline__ float sum_slots(bf16x8_t v, float acc) {
    if constexpr (std::is_same<E, f16_t>::value) {
        const f16x8_t h = __builtin_bit_cast(f16x8_t, v);
        const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 0, 1), ones, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 2, 3), ones, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 4, 5), ones, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 6, 7), ones, acc, false);
    } else {
        const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(v, v, 0, 1), ones, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(v, v, 2, 3), ones, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(v, v, 4, 5), ones, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(v, v, 6, 7), ones, acc, false);
    }
    return acc;
}

// Lane (row = lane % 32, half = lane / 32) holds, of a transposed 64 x 32 result, the values
// d = 32 dt + 8 (e / 4) + 4 half + e % 4 of its row: write them, times `mul`, as E.
template <typename E>
__device__ __forceinline__ void store_row_pieces(uint16_t* rowp, const f32x16_t* acc, float mul, int half) {
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint2 w = make_uint2(half_conv<E>::pack2(acc[dt][4 * g] * mul, acc[dt][4 * g + 1] * mul),
                                       half_conv<E>::pack2(acc[dt][4 * g + 2] * mul, acc[dt][4 * g + 3] * mul));
            *reinterpret_cast<uint2*>(rowp + 32 * dt + 8 * g + 4 * half) = w;
        }
}

// Lane l and lane l ^ 32 combined, the same result in both: v_permlane32_swap exchanges the upper half of
// its first operand with the lower half of its second, so with v in both the first comes back as the
// lower half's values in all lanes and the second as the upper half's. One VALU instruction, no LDS trip.
__device__ __forceinline__ float max_halves(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_halves(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- tile loads straight into LDS ------------------------------------------------------------------
// global_load_lds_dwordx4: lane l of the issuing wavefront writes its 16 bytes at LDS address
// M0 + 16 l, so one instruction fills 64 consecutive chunk positions of an image and the image's swizzle
// is applied on the global side: the lane fetches the chunk that belongs at its position. No staging
// registers, no LDS write instructions. The compiler does not see these loads (inline asm); the kernel
// waits for them itself (dma_wait) before the barrier that publishes the tile.

// Which chunk (row, 16-byte column) of a 64-row tile lives at chunk position p of an image.
__device__ __forceinline__ void row_image_source(int p, int& r, int& c) {
    r = p >> 3;
    c = (p & 7) ^ ((r >> 1) & 7);
}
__device__ __forceinline__ void tr_image_source(int p, int& r, int& c) {
    r = p >> 3;
    c = ((((p & 7) >> 1) ^ (r & 3)) << 1) | (p & 1);
}

// Per-thread state of the loader of one tensor: with NT threads each thread owns 512 / NT chunk
// positions of every image; `row` / `col` say which chunk of the tile belongs there.
template <int NT>
struct TileDma {
    static constexpr int kPer = 512 / NT;
    int row_r[kPer], row_c[kPer], tr_r[kPer], tr_c[kPer];
    uint32_t wave_off[kPer];  // LDS byte offset of the wavefront's 64 positions inside an image
    __device__ __forceinline__ void init(int tid) {
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int p = tid + u * NT;
            row_image_source(p, row_r[u], row_c[u]);
            tr_image_source(p, tr_r[u], tr_c[u]);
            wave_off[u] = (uint32_t)__builtin_amdgcn_readfirstlane((p >> 6) * 1024);
        }
    }
    // Tile rows row0 .. row0+63 of the [S, 64] bf16 matrix at `base` (row stride in elements); rows past
    // S read row S-1. row_img / tr_img: LDS byte addresses of the images to fill (ROW_IMAGE / TR_IMAGE
    // say which are wanted).
    template <bool ROW_IMAGE, bool TR_IMAGE>
    __device__ __forceinline__ void load(const uint16_t* base, int64_t row_stride, int row0, int S, uint32_t row_img,
                                         uint32_t tr_img) const {
        const char* g = reinterpret_cast<const char*>(base + (int64_t)row0 * row_stride);
        const int last = S - 1 - row0;
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            if (ROW_IMAGE) {
                const int r = row_r[u] < last ? row_r[u] : last;
                dma16(g, (uint32_t)((r * (int)row_stride + row_c[u] * 8) * 2), row_img + wave_off[u]);
            }
            if (TR_IMAGE) {
                const int r = tr_r[u] < last ? tr_r[u] : last;
                dma16(g, (uint32_t)((r * (int)row_stride + tr_c[u] * 8) * 2), tr_img + wave_off[u]);
            }
        }
    }
};

}  // namespace attn
}  // namespace cw
