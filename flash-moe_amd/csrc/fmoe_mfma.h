// MFMA fragment types and LDS tile helpers shared by the GEMM-shaped kernels (gfx950).
#pragma once

#include "fmoe_common.h"

namespace fmoe {

// v_mfma_f32_32x32x16_{bf16,f16}: D[32x32] += A[32x16] * B[16x32].  Lane l supplies row l%32 of A (column l%32 of B)
// and 8 consecutive k values chosen by l/32; it receives D[8*(v/4) + 4*(l/32) + v%4][l%32] in register v.
template <typename T> struct Mfma32;
template <> struct Mfma32<bf16_t> {
    using Frag = bf16x8_t;
    __device__ static f32x16_t run(Frag a, Frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma32<f16_t> {
    using Frag = f16x8_t;
    __device__ static f32x16_t run(Frag a, Frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// fp32: v_mfma_f32_32x32x2_f32, D[32x32] += A[32x2] * B[2x32]; lane l supplies A[l%32][l/32] and B[l/32][l%32], same D
// layout.  A fragment is one 16-byte LDS read like the 16-bit ones: 4 consecutive k values of the lane's row, lanes
// 0-31 from the first 16-byte chunk of a 32-byte k-step and lanes 32-63 from the second, so instruction q of a run
// multiplies the k pair {q, 4 + q} of the step - each of the 8 k values once.
template <> struct Mfma32<float> {
    using Frag = f32x4_t;
    __device__ static f32x16_t run(Frag a, Frag b, f32x16_t c) {
#pragma unroll
        for (int q = 0; q < 4; ++q) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q], b[q], c, 0, 0, 0);
        return c;
    }
};
template <typename T> constexpr int kMfmaPerRun = sizeof(T) == 4 ? 4 : 1;   // matrix instructions per Mfma32<T>::run

// v_mfma_f32_16x16x32_{bf16,f16}: D[16x16] += A[16x32] * B[32x16].  Lane l supplies row l%16 of A (column l%16 of B) and 8
// consecutive k values chosen by l/16; it receives D[4*(l/16) + v][l%16] in register v (four registers).  Under the power
// limit the chip sustains about 12 % more multiply-adds with this shape than with 32x32x16 on random data.
template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
    using Frag = bf16x8_t;
    __device__ static f32x4_t run(Frag a, Frag b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<f16_t> {
    using Frag = f16x8_t;
    __device__ static f32x4_t run(Frag a, Frag b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// What the tiled kernel needs to know about a fragment shape: FR = rows (and columns) of a fragment, kChunks = 16-byte
// pieces of a row one k-step consumes (lane l reads piece l / FR of its row l % FR), Acc with kAccRegs registers, register
// v of lane l holding D[8*(v/4) + 4*(l/FR) + v%4][l % FR] (both shapes).
template <typename T, int FR> struct MfmaShape;
template <typename T> struct MfmaShape<T, 32> {
    using Frag = typename Mfma32<T>::Frag;
    using Acc = f32x16_t;
    static constexpr int kChunks = 2, kAccRegs = 16, kInstr = kMfmaPerRun<T>;
    __device__ static Acc run(Frag a, Frag b, Acc c) { return Mfma32<T>::run(a, b, c); }
};
template <typename T> struct MfmaShape<T, 16> {
    using Frag = typename Mfma16<T>::Frag;
    using Acc = f32x4_t;
    static constexpr int kChunks = 4, kAccRegs = 4, kInstr = 1;
    __device__ static Acc run(Frag a, Frag b, Acc c) { return Mfma16<T>::run(a, b, c); }
};

// Register-staged LDS tiles: rows of 64 elements (128 bytes), 16-byte chunk index XOR-ed with (row & 7).
constexpr int kTileK = 64;
constexpr int kTileChunks = kTileK / 8;
__device__ inline int swizzled_offset(int row, int chunk) { return row * kTileK + ((chunk ^ (row & 7)) << 3); }

// Map the linear workgroup id to a tile so that each XCD gets a contiguous run of the tile order, and the tile order
// walks 8 tile-rows at a time (compact patches share A and B tiles in the XCD's L2).
__device__ inline void tile_of_block(int tiles_m, int tiles_n, int xcds, int& tm, int& tn) {
    const int nb = (int)gridDim.x;
    int t = (int)blockIdx.x;
    if (nb % xcds == 0) t = (t % xcds) * (nb / xcds) + t / xcds;
    constexpr int GM = 8;
    const int width = GM * tiles_n;
    const int group = t / width;
    const int first_m = group * GM;
    const int gsz = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    tm = first_m + (t % width) % gsz;
    tn = (t % width) / gsz;
}

}  // namespace fmoe
