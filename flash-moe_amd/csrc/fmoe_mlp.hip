// Shared SwiGLU MLP for gfx950:  out = (silu(x Wg^T) * (x Wu^T)) Wd^T [+ residual]
//
// Two launches of one MFMA GEMM  C[M,N] = A[M,K] * B[N,K]^T  (both operands K-contiguous, which is how x, the
// nn.Linear weights and the [T,I] activation are laid out, so a lane's 8 consecutive k values for one matrix
// instruction are one 16-byte LDS read):
//   1. gate/up: the B tile holds BN/2 rows of Wg and the same BN/2 rows of Wu, so each wave owns matching gate
//      and up accumulators and the epilogue writes silu(gate)*up, rounded once, to the [T,I] workspace.  The gate
//      and up products never go to memory.
//   2. down: plain epilogue, optional residual add (the routed-expert output in the block).
//
// Main kernel (gemm_dma_kernel), used when the extents are multiples of the tile: tiles go global -> LDS
// directly (global_load_lds_dwordx4, no staging registers) into NSTAGE LDS stages, issued NSTAGE-1 k-tiles
// ahead of their use; one workgroup barrier per k-tile; MFMA fragments (v_mfma_f32_16x16x32 for the 16-bit types) are
// read with 16-byte ds_reads.  An LDS row is one k-tile of one matrix row; its 16-byte chunks are XOR-swizzled with a key built
// from the row index so that the 16 lanes the 256-byte-per-clock LDS serves per cycle hit 64 different banks.
// Because a DMA load writes 64 consecutive chunks, the swizzle is applied on the global side: each lane fetches
// the chunk that belongs at its LDS position.  Workgroup ids are remapped so that each XCD (ids are dealt
// round-robin over the 8 XCDs) works on a compact patch of the tile grid and shares A/B tiles in its own L2.
//
// fp32 runs the same kernel on v_mfma_f32_32x32x2_f32: an LDS row is again 128 bytes (32 values), a fragment again one
// 16-byte read, and four matrix instructions use it.
//
// Ragged shapes take gemm_nt_kernel (register-staged, bounds-checked), in fp32 a plain FMA kernel.
#include "fmoe_common.h"
#include "fmoe_mfma.h"

namespace fmoe {
namespace {

constexpr int kGemmThreads = 256;
constexpr int BK = kTileK;        // k extent of a register-staged LDS tile (elements)
constexpr int kChunksPerRow = kTileChunks;

enum Epilogue { kEpiSwiGLU = 0, kEpiPlain = 1, kEpiDual = 2 };   // Dual: the product in T and, through R, in fp32
template <bool B> struct Flag { static constexpr bool value = B; };

template <typename T, int BM, int BN, int EPI>
__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(
    const T* __restrict__ A, const T* __restrict__ B0, const T* __restrict__ B1, T* __restrict__ C,
    const T* __restrict__ R, int M, int N, int K, int tiles_m, int tiles_n, int xcds) {
    using Frag = typename Mfma32<T>::Frag;
    constexpr int WM = BM / 2, WN = BN / 2;        // per-wave tile
    constexpr int MF = WM / 32, NF = WN / 32;      // 32x32 fragments per wave
    constexpr int A_CHUNKS = BM * kChunksPerRow / kGemmThreads;
    constexpr int B_CHUNKS = BN * kChunksPerRow / kGemmThreads;
    constexpr int BN_OUT = (EPI == kEpiSwiGLU) ? BN / 2 : BN;   // output columns per tile

    __shared__ __attribute__((aligned(16))) T As[BM * BK];
    __shared__ __attribute__((aligned(16))) T Bs[BN * BK];

    int tm, tn;
    tile_of_block(tiles_m, tiles_n, xcds, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN_OUT;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    u32x4_t ra[A_CHUNKS], rb[B_CHUNKS];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int it = 0; it < A_CHUNKS; ++it) {
            const int q = it * kGemmThreads + tid;
            const int row = q / kChunksPerRow, ch = q % kChunksPerRow;
            const int gm = m0 + row, gk = k0 + ch * 8;
            ra[it] = (gm < M && gk < K) ? *reinterpret_cast<const u32x4_t*>(A + (int64_t)gm * K + gk) : zero4;
        }
#pragma unroll
        for (int it = 0; it < B_CHUNKS; ++it) {
            const int q = it * kGemmThreads + tid;
            const int row = q / kChunksPerRow, ch = q % kChunksPerRow;
            const int gk = k0 + ch * 8;
            const T* base;
            int gn;
            if (EPI == kEpiSwiGLU) {
                const bool is_up = row >= BN / 2;
                base = is_up ? B1 : B0;
                gn = n0 + (is_up ? row - BN / 2 : row);
            } else {
                base = B0;
                gn = n0 + row;
            }
            rb[it] = (gn < N && gk < K) ? *reinterpret_cast<const u32x4_t*>(base + (int64_t)gn * K + gk) : zero4;
        }
    };
    auto store_lds = [&]() {
#pragma unroll
        for (int it = 0; it < A_CHUNKS; ++it) {
            const int q = it * kGemmThreads + tid;
            *reinterpret_cast<u32x4_t*>(&As[swizzled_offset(q / kChunksPerRow, q % kChunksPerRow)]) = ra[it];
        }
#pragma unroll
        for (int it = 0; it < B_CHUNKS; ++it) {
            const int q = it * kGemmThreads + tid;
            *reinterpret_cast<u32x4_t*>(&Bs[swizzled_offset(q / kChunksPerRow, q % kChunksPerRow)]) = rb[it];
        }
    };

    f32x16_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
        for (int j = 0; j < NF; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // LDS row of this lane inside fragment f of the wave's A / B sub-tile
    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;   // which 8 of the 16 k values of one MFMA this lane supplies
    int b_row[NF];
#pragma unroll
    for (int j = 0; j < NF; ++j) {
        if (EPI == kEpiSwiGLU)
            b_row[j] = (j < NF / 2) ? wn * (BN / 4) + j * 32 + frag_row
                                    : BN / 2 + wn * (BN / 4) + (j - NF / 2) * 32 + frag_row;
        else
            b_row[j] = wn * WN + j * 32 + frag_row;
    }

    const int k_tiles = (K + BK - 1) / BK;
    load_global(0);
    store_lds();
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
        if (kt + 1 < k_tiles) load_global((kt + 1) * BK);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int chunk = ks * 2 + frag_half;
            Frag fa[MF], fb[NF];
#pragma unroll
            for (int i = 0; i < MF; ++i)
                fa[i] = *reinterpret_cast<const Frag*>(&As[swizzled_offset(wm * WM + i * 32 + frag_row, chunk)]);
#pragma unroll
            for (int j = 0; j < NF; ++j) fb[j] = *reinterpret_cast<const Frag*>(&Bs[swizzled_offset(b_row[j], chunk)]);
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
                for (int j = 0; j < NF; ++j) acc[i][j] = Mfma32<T>::run(fa[i], fb[j], acc[i][j]);
        }
        __syncthreads();
        if (kt + 1 < k_tiles) {
            store_lds();
            __syncthreads();
        }
    }

    // D fragment layout of v_mfma_f32_32x32x*: lane l, register v holds
    //   row = 8*(v/4) + 4*(l/32) + (v%4)   (A / M index),   col = l%32   (B / N index)
    if (EPI == kEpiSwiGLU) {
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int j = 0; j < NF / 2; ++j) {
                const int col = n0 + wn * (BN / 4) + j * 32 + frag_row;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * frag_half + (v % 4);
                    if (row < M && col < N) {
                        const float g = acc[i][j][v], u = acc[i][j + NF / 2][v];
                        C[(int64_t)row * N + col] = Elem<T>::from_f32(silu_f32(g) * u);
                        if (R != nullptr) {   // planes [0] and [1] of a [2, M, N] buffer keep the two products
                            const_cast<T*>(R)[(int64_t)row * N + col] = Elem<T>::from_f32(g);
                            const_cast<T*>(R)[((int64_t)M + row) * N + col] = Elem<T>::from_f32(u);
                        }
                    }
                }
            }
    } else {
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int j = 0; j < NF; ++j) {
                const int col = n0 + wn * WN + j * 32 + frag_row;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * frag_half + (v % 4);
                    if (row < M && col < N) {
                        float r = acc[i][j][v];
                        if (R != nullptr) r += Elem<T>::to_f32(R[(int64_t)row * N + col]);
                        C[(int64_t)row * N + col] = Elem<T>::from_f32(r);
                    }
                }
            }
    }
}


// ------------------------------------------------------------------------------------------------------------
// LDS-DMA pipelined kernel.  WAVES_M x WAVES_N waves, each (BM/WAVES_M) x (BN/WAVES_N); BKT = k extent of a stage.
// ------------------------------------------------------------------------------------------------------------
// FR: fragment shape (32: v_mfma_f32_32x32x16 / 32x32x2; 16: v_mfma_f32_16x16x32).  SPLIT: a k-step's A fragments are read and
// multiplied in SPLIT parts (its B fragments stay for the whole k-step), which halves the registers the read-ahead needs.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int BKT, int NSTAGE, int EPI, int PF, int FR = 32, int SPLIT = 1>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_dma_kernel(
    const T* __restrict__ A, const T* __restrict__ B0, const T* __restrict__ B1, T* __restrict__ C,
    const T* __restrict__ R, int M, int N, int K, int tiles_m, int tiles_n, int xcds) {
    using Shape = MfmaShape<T, FR>;
    using Frag = typename Shape::Frag;
    using Acc = typename Shape::Acc;
    constexpr int NV = Shape::kAccRegs;
    constexpr int NWAVES = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, MF = WM / FR, NF = WN / FR;
    constexpr int EPC = 16 / (int)sizeof(T);        // elements per 16-byte chunk
    constexpr int CPR = BKT / EPC;                  // 16-byte chunks per LDS row
    constexpr int RPI = 64 / CPR;                   // rows one wave-wide DMA load covers
    constexpr int ROWS_PER_IT = NWAVES * RPI;       // rows all waves cover per DMA round
    constexpr int STAGE = (BM + BN) * BKT;          // elements per stage
    constexpr int KSTEPS = BKT / (Shape::kChunks * EPC);   // a k-step is kChunks 16-byte pieces of a row: one per lane group
    constexpr int SPK = KSTEPS * SPLIT;             // steps (a part of a k-step's A fragments against all its B fragments) per k-tile
    constexpr int MFS = MF / SPLIT;
    static_assert(MF % SPLIT == 0 && WM % FR == 0 && WN % FR == 0, "fragments tile the wave tile");
    constexpr int ROW_SHIFT = (CPR == 8) ? 1 : 2;   // log2(rows per 256 bytes)
    constexpr int BN_OUT = (EPI == kEpiSwiGLU) ? BN / 2 : BN;
    constexpr int A_ROUNDS = BM / ROWS_PER_IT, B_ROUNDS = BN / ROWS_PER_IT;
    constexpr int DMA_PER_TILE = A_ROUNDS + B_ROUNDS;
    static_assert(CPR == 4 || CPR == 8, "stage depth: LDS rows of 64 or 128 bytes");
    static_assert(ROWS_PER_IT % 16 == 0 && BM % ROWS_PER_IT == 0 && BN % ROWS_PER_IT == 0, "DMA rounds");
    static_assert(EPI != kEpiSwiGLU || ((BN / 2) % ROWS_PER_IT == 0 && NF % 2 == 0), "gate/up split");
    static_assert((NSTAGE - 2) * DMA_PER_TILE < 64, "vmcnt range");

    __shared__ __attribute__((aligned(1024))) T lds[NSTAGE * STAGE];

    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int num_tiles = tiles_m * tiles_n;

    // DMA: the lane's LDS position is row (round*ROWS_PER_IT + wave*RPI + lrow), physical chunk lp; it holds the
    // logical chunk lp ^ key(row), key(row) = (row >> ROW_SHIFT) & (CPR-1).  ROWS_PER_IT is a multiple of 16, so the
    // key does not depend on the round and one element offset per lane serves every load.
    const int lrow = lane / CPR, lp = lane % CPR;
    const int key_dma = ((wave * RPI + lrow) >> ROW_SHIFT) & (CPR - 1);
    const uint32_t lane_off = (uint32_t)(lrow * K + (lp ^ key_dma) * EPC) * (uint32_t)sizeof(T);   // bytes
    // A rows beyond M (a ragged last tile row) are read from row M-1 instead: one byte offset per DMA round, set per
    // tile.  What the MFMAs make of those rows is never stored (the epilogue's buffer stores are bounds-checked).
    uint32_t a_lane_off[A_ROUNDS];
    const T *a_src, *b_src0, *b_src1 = nullptr;
    int m0, n0;
    // The workgroup is persistent: it takes tiles t, t + gridDim.x, ...  Each XCD (workgroup id mod 8) gets a contiguous
    // run of the tile order, walked 8 tile-rows at a time so that a compact patch shares A and B tiles in the XCD's L2.
    auto set_tile = [&](int t) {
        if (num_tiles % xcds == 0) t = (t % xcds) * (num_tiles / xcds) + t / xcds;
        constexpr int GM = 8;
        const int width = GM * tiles_n, group = t / width, first_m = group * GM;
        const int gsz = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
        m0 = (first_m + (t % width) % gsz) * BM;
        n0 = ((t % width) / gsz) * BN_OUT;
        a_src = A + (int64_t)m0 * K;                     // wave-uniform; the lane's part is the 32-bit a_lane_off[r]
#pragma unroll
        for (int r = 0; r < A_ROUNDS; ++r) {
            int row = r * ROWS_PER_IT + wave * RPI + lrow;
            row = m0 + row < M ? row : M - 1 - m0;
            a_lane_off[r] = (uint32_t)(row * K + (lp ^ key_dma) * EPC) * (uint32_t)sizeof(T);
        }
        b_src0 = B0 + (int64_t)(n0 + wave * RPI) * K;
        if (EPI == kEpiSwiGLU) b_src1 = B1 + (int64_t)(n0 + wave * RPI) * K;
    };
    auto issue = [&](int kt, T* stage) {
        const int k0 = kt * BKT;
#pragma unroll
        for (int r = 0; r < A_ROUNDS; ++r)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)((const char*)(a_src + k0) + a_lane_off[r]),
                (__attribute__((address_space(3))) void*)(stage + (r * ROWS_PER_IT + wave * RPI) * BKT), 16, 0, 0);
#pragma unroll
        for (int r = 0; r < B_ROUNDS; ++r) {
            const T* src;
            if (EPI == kEpiSwiGLU && r >= B_ROUNDS / 2) src = b_src1 + (int64_t)(r - B_ROUNDS / 2) * ROWS_PER_IT * K + k0;
            else src = b_src0 + (int64_t)r * ROWS_PER_IT * K + k0;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)((const char*)src + lane_off),
                (__attribute__((address_space(3))) void*)(stage + BM * BKT + (r * ROWS_PER_IT + wave * RPI) * BKT), 16, 0, 0);
        }
    };

    // Fragment rows of a lane are (multiple of FR) + frow: the swizzle key is the same for all of them, so the
    // address is (row base + one per-k-step offset) + an immediate per fragment.
    const int frow = lane % FR, fhalf = lane / FR;       // fhalf: which 16-byte piece of a k-step the lane supplies
    const int key_f = (frow >> ROW_SHIFT) & (CPR - 1);
    const int a_row_bytes = (wm * WM + frow) * BKT * (int)sizeof(T);
    int b_row_bytes[NF];
#pragma unroll
    for (int j = 0; j < NF; ++j) {
        int row;
        if (EPI == kEpiSwiGLU) row = (j < NF / 2) ? wn * (WN / 2) + j * FR : BN / 2 + wn * (WN / 2) + (j - NF / 2) * FR;
        else row = wn * WN + j * FR;
        b_row_bytes[j] = (BM + row + frow) * BKT * (int)sizeof(T);
    }
    int pc[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) pc[ks] = ((ks * Shape::kChunks + fhalf) ^ key_f) << 4;

    const int k_tiles = K / BKT;
    int tile = (int)blockIdx.x;
    if (tile >= num_tiles) return;
    set_tile(tile);
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s)
        if (s < k_tiles) issue(s, lds + s * STAGE);

    // Fragments of step q+PF are read from LDS while the MFMAs of step q run (PF+1 register buffers for the A parts; B
    // fragments are read with the first part of their k-step); the read-ahead crosses k-tile boundaries, so the barrier
    // that publishes the next stage sits PF steps before the end of a k-tile and the matrix pipe always has work queued
    // while a wave waits.
    constexpr int RING = PF + 1;
    constexpr int RINGB = SPLIT == 1 ? RING : 2;
    static_assert(SPK % RING == 0 && PF >= 1 && PF < SPK + 1, "fragment buffers rotate with period RING");
    static_assert(SPLIT == 1 || (PF <= SPLIT && KSTEPS % 2 == 0), "with split k-steps at most the next k-step's B fragments are in flight");
    Frag fa[RING][MFS], fb[RINGB][NF];
    auto b_slot = [](int q) { return SPLIT == 1 ? q % RING : (q / SPLIT) % 2; };     // q: step inside the k-tile (may exceed SPK by PF)
    auto read_frags = [&](const char* stage, int q, Frag (&a)[MFS], Frag (&b)[NF]) {
        const int ks = q / SPLIT, part = q % SPLIT;
#pragma unroll
        for (int i = 0; i < MFS; ++i)
            a[i] = *reinterpret_cast<const Frag*>(stage + a_row_bytes + pc[ks] + (part * MFS + i) * FR * BKT * (int)sizeof(T));
        if (part == 0) {
#pragma unroll
            for (int j = 0; j < NF; ++j) b[j] = *reinterpret_cast<const Frag*>(stage + b_row_bytes[j] + pc[ks]);
        }
    };
    // Entering k-tile kt (kt = 0: from the tile prologue): my share of its stage has landed once at most the loads of
    // the NSTAGE-2 younger k-tiles are outstanding; my reads of the stage that is overwritten next are complete (all
    // reads of k-tile kt-1 have been issued by then); after the barrier both hold for every wave, so the load of k-tile
    // kt+NSTAGE-1 can go into the stage kt-1 used.
    auto enter_k_tile = [&](int kt) {
        constexpr int kKeep = (NSTAGE - 2) * DMA_PER_TILE;
        if (kt + NSTAGE - 2 < k_tiles) __builtin_amdgcn_s_waitcnt(0x0070 | (kKeep & 0xF) | ((kKeep >> 4) << 14));
        else __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
        if (kt + NSTAGE - 1 < k_tiles) issue(kt + NSTAGE - 1, lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE);
    };
    while (true) {
        Acc acc[MF][NF];
#pragma unroll
        for (int i = 0; i < MF; ++i)
#pragma unroll
            for (int j = 0; j < NF; ++j)
#pragma unroll
                for (int v = 0; v < NV; ++v) acc[i][j][v] = 0.0f;

        enter_k_tile(0);
#pragma unroll
        for (int s = 0; s < PF; ++s) read_frags(reinterpret_cast<const char*>(lds), s, fa[s % RING], fb[b_slot(s)]);
        // the last k-tile has no successor to read ahead into: it is a separate copy of the body, so that no branch
        // merges a path with reads in flight into the MFMA sequence
        auto k_tile_body = [&](int kt, auto last_tag) {
            constexpr bool kLast = decltype(last_tag)::value;
            const char* stage = reinterpret_cast<const char*>(lds + (kt % NSTAGE) * STAGE);
            const char* next_stage = reinterpret_cast<const char*>(lds + ((kt + 1) % NSTAGE) * STAGE);
#pragma unroll
            for (int q = 0; q < SPK; ++q) {
                const int nxt = q + PF;
                constexpr int kMfmas = MFS * NF;     // runs of Shape::kInstr instructions
                const bool reads = nxt < SPK || !kLast;
                const int n_reads = MFS + ((nxt % SPLIT) == 0 ? NF : 0);
                __builtin_amdgcn_sched_barrier(0);
                if (nxt < SPK) {
                    read_frags(stage, nxt, fa[nxt % RING], fb[b_slot(nxt)]);
                } else if (!kLast) {
                    if (nxt == SPK) {
                        enter_k_tile(kt + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    read_frags(next_stage, nxt - SPK, fa[nxt % RING], fb[b_slot(nxt)]);
                }
                const int part = q % SPLIT;
#pragma unroll
                for (int i = 0; i < MFS; ++i)
#pragma unroll
                    for (int j = 0; j < NF; ++j)
                        acc[part * MFS + i][j] = Shape::run(fa[q % RING][i], fb[b_slot(q)][j], acc[part * MFS + i][j]);
                // issue order: the LDS reads spread evenly behind the MFMAs
                constexpr int kPer = (MFS + NF + kMfmas - 1) / kMfmas;
#pragma unroll
                for (int m = 0; m < kMfmas; ++m) {
                    __builtin_amdgcn_sched_group_barrier(0x008, Shape::kInstr, 0);
                    if (reads && m * kPer < n_reads) __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);
                }
            }
        };
        for (int kt = 0; kt + 1 < k_tiles; ++kt) k_tile_body(kt, Flag<false>{});
        k_tile_body(k_tiles - 1, Flag<true>{});
        __builtin_amdgcn_sched_barrier(0);

        // start the next tile's first stages before this tile's epilogue, so that its global-load latency is covered
        const int out_m0 = m0, out_n0 = n0;
        const int next = tile + (int)gridDim.x;
        if (next < num_tiles) {
            set_tile(next);
            __builtin_amdgcn_s_barrier();     // every wave has consumed its reads of the last stage
#pragma unroll
            for (int s = 0; s < NSTAGE - 1; ++s)
                if (s < k_tiles) issue(s, lds + s * STAGE);
        }

        // D fragment layout (both shapes): lane l, register v holds
        //   row = 8*(v/4) + 4*(l/FR) + (v%4)   (A / M index),   col = l%FR   (B / N index)
        // Buffer addressing: a wave-uniform descriptor of the rows from the wave's first one on, a scalar byte offset
        // per (fragment, register) and one 32-bit byte offset per lane - no vector address arithmetic per element.
        const int lane_bytes = ((4 * fhalf) * N + frow) * (int)sizeof(T);
        const int64_t wave_off = (int64_t)(out_m0 + wm * WM) * N + out_n0 + wn * ((EPI == kEpiSwiGLU) ? WN / 2 : WN);
        const int64_t span = ((int64_t)M * N - wave_off) * (int64_t)sizeof(T);
        // a wave whose rows all lie beyond M gets an empty descriptor: every access of it is dropped
        const int span32 = (int)(span < 0 ? 0 : (span < 0x7FFFFFFFll ? span : 0x7FFFFFFFll));
        auto c_rsrc = __builtin_amdgcn_make_buffer_rsrc(C + wave_off, 0, span32, 0x00020000);
        auto store_to = [&](auto rsrc, int uni_bytes, float value) {
            if constexpr (sizeof(T) == 4) {
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, value), rsrc, lane_bytes, uni_bytes, 0);
            } else {
                const T t = Elem<T>::from_f32(value);
                __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(short, t), rsrc, lane_bytes, uni_bytes, 0);
            }
        };
        auto store_elem = [&](int uni_bytes, float value) { store_to(c_rsrc, uni_bytes, value); };
        // 16-bit outputs round once, so the fast reciprocal's last-bit error is invisible; fp32 divides
        auto silu = [](float v) { return sizeof(T) == 4 ? silu_f32(v) : silu_fast_f32(v); };
        // element offset of (fragment i, fragment column j, register v) from the wave's first output element
        auto elem_at = [&](int i, int j, int v) { return (i * FR + 8 * (v / 4) + (v % 4)) * N + j * FR; };
        if (EPI == kEpiSwiGLU) {
            if (R != nullptr) {
                // keep the gate and up products for a backward pass: planes [0] and [1] of a [2, M, N] buffer
                T* planes = const_cast<T*>(R);
                auto g_rsrc = __builtin_amdgcn_make_buffer_rsrc(planes + wave_off, 0, span32, 0x00020000);
                auto u_rsrc = __builtin_amdgcn_make_buffer_rsrc(planes + (int64_t)M * N + wave_off, 0, span32, 0x00020000);
#pragma unroll
                for (int i = 0; i < MF; ++i)
#pragma unroll
                    for (int j = 0; j < NF / 2; ++j)
#pragma unroll
                        for (int v = 0; v < NV; ++v) {
                            const int uni = elem_at(i, j, v) * (int)sizeof(T);
                            store_to(g_rsrc, uni, acc[i][j][v]);
                            store_to(u_rsrc, uni, acc[i][j + NF / 2][v]);
                        }
            }
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
                for (int j = 0; j < NF / 2; ++j)
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        store_elem(elem_at(i, j, v) * (int)sizeof(T), silu(acc[i][j][v]) * acc[i][j + NF / 2][v]);
        } else if (EPI == kEpiDual) {
            // R points at an fp32 [M, N] buffer that receives the unrounded sums next to the rounded ones in C
            float* out32 = reinterpret_cast<float*>(const_cast<T*>(R));
            const int64_t span_f = ((int64_t)M * N - wave_off) * 4;
            const int span32_f = (int)(span_f < 0 ? 0 : (span_f < 0x7FFFFFFFll ? span_f : 0x7FFFFFFFll));
            auto f_rsrc = __builtin_amdgcn_make_buffer_rsrc(out32 + wave_off, 0, span32_f, 0x00020000);
            const int lane_bytes_f = ((4 * fhalf) * N + frow) * 4;
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
                for (int j = 0; j < NF; ++j)
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const int at = elem_at(i, j, v);
                        const float sum = acc[i][j][v];      // a scalar copy: the bit cast below must not see a vector element
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, sum), f_rsrc, lane_bytes_f, at * 4, 0);
                        store_elem(at * (int)sizeof(T), sum);
                    }
        } else {
            auto r_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(R != nullptr ? R + wave_off : C), 0,
                                                            R != nullptr ? span32 : 0, 0x00020000);   // no residual: reads give 0
#pragma unroll
            for (int i = 0; i < MF; ++i)
#pragma unroll
                for (int j = 0; j < NF; ++j) {
                    float res[NV];
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const int uni = elem_at(i, j, v) * (int)sizeof(T);
                        if constexpr (sizeof(T) == 4) {
                            res[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_rsrc, lane_bytes, uni, 0));
                        } else {
                            const short raw = __builtin_amdgcn_raw_buffer_load_b16(r_rsrc, lane_bytes, uni, 0);
                            res[v] = Elem<T>::to_f32(__builtin_bit_cast(T, raw));
                        }
                    }
#pragma unroll
                    for (int v = 0; v < NV; ++v) store_elem(elem_at(i, j, v) * (int)sizeof(T), acc[i][j][v] + res[v]);
                }
        }
        if (next >= num_tiles) break;
        tile = next;
    }
}

// fp32 with ragged extents or unaligned tensors (not a tuned kernel): 64x64 tile, 16-deep LDS slabs, 4x4 outputs
// per thread, plain FMA.
template <int EPI>
__global__ __launch_bounds__(256) void sgemm_nt_kernel(const float* __restrict__ A, const float* __restrict__ B0,
                                                       const float* __restrict__ B1, float* __restrict__ C,
                                                       const float* __restrict__ R, int M, int N, int K) {
    constexpr int TS = 64, KS = 16;
    __shared__ float As[KS][TS + 1];
    __shared__ float Bg[KS][TS + 1];
    __shared__ float Bu[(EPI == kEpiSwiGLU) ? KS : 1][TS + 1];
    const int m0 = blockIdx.y * TS, n0 = blockIdx.x * TS;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    float accg[4][4] = {}, accu[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += KS) {
        for (int q = threadIdx.x; q < TS * KS; q += 256) {
            const int r = q / KS, kk = q % KS;
            const int gk = k0 + kk;
            As[kk][r] = (m0 + r < M && gk < K) ? A[(int64_t)(m0 + r) * K + gk] : 0.0f;
            Bg[kk][r] = (n0 + r < N && gk < K) ? B0[(int64_t)(n0 + r) * K + gk] : 0.0f;
            if (EPI == kEpiSwiGLU) Bu[kk][r] = (n0 + r < N && gk < K) ? B1[(int64_t)(n0 + r) * K + gk] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            float a[4], g[4], u[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[j] = Bg[kk][tx * 4 + j];
                u[j] = (EPI == kEpiSwiGLU) ? Bu[kk][tx * 4 + j] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    accg[i][j] = __builtin_fmaf(a[i], g[j], accg[i][j]);
                    if (EPI == kEpiSwiGLU) accu[i][j] = __builtin_fmaf(a[i], u[j], accu[i][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + ty * 4 + i, col = n0 + tx * 4 + j;
            if (row < M && col < N) {
                float r = (EPI == kEpiSwiGLU) ? silu_f32(accg[i][j]) * accu[i][j] : accg[i][j];
                if (EPI == kEpiPlain && R != nullptr) r += R[(int64_t)row * N + col];
                if (EPI == kEpiSwiGLU && R != nullptr) {
                    const_cast<float*>(R)[(int64_t)row * N + col] = accg[i][j];
                    const_cast<float*>(R)[((int64_t)M + row) * N + col] = accu[i][j];
                }
                C[(int64_t)row * N + col] = r;
            }
        }
}

template <typename T, int BM, int BN, int EPI>
void launch_gemm(const T* A, const T* B0, const T* B1, T* C, const T* R, int M, int N, int K, hipStream_t stream) {
    constexpr int BN_OUT = (EPI == kEpiSwiGLU) ? BN / 2 : BN;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN_OUT - 1) / BN_OUT;
    hipLaunchKernelGGL((gemm_nt_kernel<T, BM, BN, EPI>), dim3((unsigned)(tiles_m * tiles_n)), dim3(kGemmThreads), 0,
                       stream, A, B0, B1, C, R, M, N, K, tiles_m, tiles_n, chip_info().xcds);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int BKT, int NSTAGE, int EPI, int PF, int FR = 32, int SPLIT = 1>
void launch_gemm_dma(const T* A, const T* B0, const T* B1, T* C, const T* R, int M, int N, int K, hipStream_t stream) {
    constexpr int BN_OUT = (EPI == kEpiSwiGLU) ? BN / 2 : BN;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = N / BN_OUT;      // a ragged last row of tiles is allowed
    // persistent workgroups: as many as are resident at once (LDS-limited), a multiple of 8 so that the XCD patches hold
    constexpr int kStageBytes = (BM + BN) * BKT * (int)sizeof(T) * NSTAGE;
    constexpr int kPerCu = (160 * 1024 / kStageBytes) < 1 ? 1 : ((160 * 1024 / kStageBytes) > 2 ? 2 : (160 * 1024 / kStageBytes));
    const int total = tiles_m * tiles_n;
    const ChipInfo& chip = chip_info();
    const int resident = chip.cus * kPerCu;
    const int grid = total < resident ? total : resident;
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, WAVES_M, WAVES_N, BKT, NSTAGE, EPI, PF, FR, SPLIT>), dim3((unsigned)grid),
                       dim3(WAVES_M * WAVES_N * 64), 0, stream, A, B0, B1, C, R, M, N, K, tiles_m, tiles_n, chip.xcds);
}

// k extent of one LDS stage of the DMA kernel: 128 bytes of a row for every element type
template <typename T> constexpr int kStageK = 128 / (int)sizeof(T);
// 16-bit products run on v_mfma_f32_16x16x32 (more multiply-adds per joule than 32x32x16, which is what bounds these
// kernels); a k-step is then half a stage, so the read-ahead is one step, and the 256 x 256 tile reads a k-step's A
// fragments in four parts to stay inside 256 registers per wave (in two parts it spills 24).  fp32 keeps 32x32x2.
template <typename T> constexpr int kFragRows = sizeof(T) == 2 ? 16 : 32;
template <typename T> constexpr int kBigSplit = sizeof(T) == 2 ? 4 : 1;
template <typename T> constexpr int kSmallAhead = sizeof(T) == 2 ? 1 : 3;

// Ragged shapes: the bounds-checked kernels (register-staged MFMA for 16-bit, FMA for fp32).
template <typename T, int EPI>
void launch_ragged(const T* A, const T* B0, const T* B1, T* C, const T* R, int M, int N, int K, hipStream_t stream) {
    if constexpr (sizeof(T) == 4)
        hipLaunchKernelGGL((sgemm_nt_kernel<EPI>), dim3((N + 63) / 64, (M + 63) / 64), dim3(256), 0, stream, A, B0, B1, C, R, M, N, K);
    else
        launch_gemm<T, 128, 128, EPI>(A, B0, B1, C, R, M, N, K, stream);
}

// Tile choice: 256-wide tiles (8 waves, two per SIMD) halve the L2 -> LDS traffic per MFMA but need one per CU to
// occupy the chip; otherwise 128x128 tiles of 4 waves, which read half a k-tile of fragments ahead (a whole one in fp32): one
// workgroup per CU with four stages in flight when every tile gets a CU of its own, two per CU with two stages else.
template <typename T, int EPI>
void launch_small_tiles(const T* A, const T* B0, const T* B1, T* C, const T* R, int M, int N, int K, int64_t tiles,
                        hipStream_t stream) {
    constexpr int KT = kStageK<T>;
    if (tiles <= chip_info().cus) launch_gemm_dma<T, 128, 128, 2, 2, KT, 4, EPI, kSmallAhead<T>, kFragRows<T>>(A, B0, B1, C, R, M, N, K, stream);
    else launch_gemm_dma<T, 128, 128, 2, 2, KT, 2, EPI, kSmallAhead<T>, kFragRows<T>>(A, B0, B1, C, R, M, N, K, stream);
}

// Few tokens: 64-row tiles (wave tiles of 32 x 64 or 32 x 32), so that a batch of a few hundred tokens still gives
// every CU a tile.  N_OUT: output columns of a tile.
template <typename T, int EPI>
void launch_narrow_tiles(const T* A, const T* B0, const T* B1, T* C, const T* R, int M, int N, int K, hipStream_t stream) {
    if (EPI == kEpiPlain && (int64_t)((M + 63) / 64) * (N / 128) < chip_info().cus && N % 64 == 0)
        launch_gemm_dma<T, 64, 64, 2, 2, kStageK<T>, 4, kEpiPlain, kSmallAhead<T>, kFragRows<T>>(A, B0, B1, C, R, M, N, K, stream);
    else
        launch_gemm_dma<T, 64, 128, 2, 2, kStageK<T>, 4, EPI, kSmallAhead<T>, kFragRows<T>>(A, B0, B1, C, R, M, N, K, stream);
}

template <typename T>
int gate_up_tiled(const void* x, const void* wg, const void* wu, int M, int H, int I, void* h, void* saved, hipStream_t stream) {
    const T *A = (const T*)x, *G = (const T*)wg, *U = (const T*)wu, *S = (const T*)saved;
    // the DMA kernel moves 16-byte pieces (fp32 callers need not align their tensors; those take the ragged kernel)
    const bool k_ok = H % kStageK<T> == 0 && aligned16(x) && aligned16(wg) && aligned16(wu);
    if (k_ok && I % 128 == 0 && (int64_t)((M + 255) / 256) * (I / 128) >= chip_info().cus)
        launch_gemm_dma<T, 256, 256, 2, 4, kStageK<T>, 2, kEpiSwiGLU, 1, kFragRows<T>, kBigSplit<T>>(A, G, U, (T*)h, S, M, I, H, stream);
    else if (k_ok && I % 64 == 0 && (int64_t)((M + 127) / 128) * (I / 64) >= chip_info().cus)
        launch_small_tiles<T, kEpiSwiGLU>(A, G, U, (T*)h, S, M, I, H, (int64_t)((M + 127) / 128) * (I / 64), stream);
    else if (k_ok && I % 64 == 0)
        launch_narrow_tiles<T, kEpiSwiGLU>(A, G, U, (T*)h, S, M, I, H, stream);
    else
        launch_ragged<T, kEpiSwiGLU>(A, G, U, (T*)h, S, M, I, H, stream);
    FMOE_CHECK_LAUNCH("fmoe_mlp(gate/up)");
    return FMOE_OK;
}

template <typename T>
int down_tiled(const void* h, const void* wd, int M, int H, int I, const void* residual, void* out, hipStream_t stream) {
    const T *A = (const T*)h, *W = (const T*)wd, *R = (const T*)residual;
    const bool k_ok = I % kStageK<T> == 0 && aligned16(h) && aligned16(wd);
    if (k_ok && H % 256 == 0 && (int64_t)((M + 255) / 256) * (H / 256) >= chip_info().cus)
        launch_gemm_dma<T, 256, 256, 2, 4, kStageK<T>, 2, kEpiPlain, 1, kFragRows<T>, kBigSplit<T>>(A, W, nullptr, (T*)out, R, M, H, I, stream);
    else if (k_ok && H % 128 == 0 && (int64_t)((M + 127) / 128) * (H / 128) >= chip_info().cus)
        launch_small_tiles<T, kEpiPlain>(A, W, nullptr, (T*)out, R, M, H, I, (int64_t)((M + 127) / 128) * (H / 128), stream);
    else if (k_ok && H % 128 == 0)
        launch_narrow_tiles<T, kEpiPlain>(A, W, nullptr, (T*)out, R, M, H, I, stream);
    else
        launch_ragged<T, kEpiPlain>(A, W, nullptr, (T*)out, R, M, H, I, stream);
    FMOE_CHECK_LAUNCH("fmoe_mlp(down)");
    return FMOE_OK;
}

}  // namespace

// C[M,N] = A[M,K] * B[N,K]^T in the 16-bit dtype and in fp32 (the same sums before rounding), on 256 x 256 tiles of the
// DMA kernel: for products large enough to give every compute unit a tile (the router's gate product for tens of thousands
// of tokens).  The k order of the sums is that of every other kernel here: ascending, 16 values per matrix instruction.
bool gemm_nt_dual_usable(int64_t M, int N, int K) {
    return M > 0 && M < (1ll << 31) && N % 256 == 0 && K % 64 == 0 && ((M + 255) / 256) * (int64_t)(N / 256) >= chip_info().cus;
}
int gemm_nt_dual(const void* A, const void* B, void* C, float* C32, int M, int N, int K, int dtype, hipStream_t stream) {
    if (dtype == FMOE_BF16)
        launch_gemm_dma<bf16_t, 256, 256, 2, 4, 64, 2, kEpiDual, 1>((const bf16_t*)A, (const bf16_t*)B, nullptr, (bf16_t*)C,
                                                                    (const bf16_t*)C32, M, N, K, stream);
    else
        launch_gemm_dma<f16_t, 256, 256, 2, 4, 64, 2, kEpiDual, 1>((const f16_t*)A, (const f16_t*)B, nullptr, (f16_t*)C,
                                                                   (const f16_t*)C32, M, N, K, stream);
    FMOE_CHECK_LAUNCH("gate product (tiled)");
    return FMOE_OK;
}

namespace {

int check_mlp_shape(const char* who, int64_t T_, int H, int I, int dtype) {
    FMOE_REQUIRE(dtype_ok(dtype), FMOE_ERR_BAD_DTYPE, "%s: unknown dtype %d", who, dtype);
    FMOE_REQUIRE(T_ >= 0 && H > 0 && I > 0, FMOE_ERR_BAD_SHAPE, "%s: bad shape T=%lld H=%d I=%d", who, (long long)T_, H, I);
    FMOE_REQUIRE(T_ < (1ll << 31), FMOE_ERR_UNSUPPORTED, "%s: T=%lld >= 2^31", who, (long long)T_);
    if (dtype != FMOE_F32)
        FMOE_REQUIRE(H % 8 == 0 && I % 8 == 0, FMOE_ERR_ALIGNMENT,
                     "%s: hidden=%d and intermediate=%d must be multiples of 8 (16-byte rows)", who, H, I);
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" size_t fmoe_mlp_workspace_bytes(int64_t num_tokens, int hidden, int intermediate, int dtype) {
    (void)hidden;
    if (num_tokens <= 0 || intermediate <= 0 || !fmoe::dtype_ok(dtype)) return 0;
    return fmoe::round_up((size_t)num_tokens * (size_t)intermediate * fmoe::dtype_size(dtype), 256);
}

namespace fmoe {
namespace {
int mlp_gate_up_impl(const char* who, const void* x, const void* gate_w, const void* up_w, int64_t num_tokens, int hidden,
                     int intermediate, int dtype, void* act, void* saved, void* stream) {
    clear_error();
    if (int rc = check_mlp_shape(who, num_tokens, hidden, intermediate, dtype)) return rc;
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(x && gate_w && up_w && act, FMOE_ERR_NULL_POINTER, "%s: null tensor pointer", who);
    FMOE_REQUIRE(dtype == FMOE_F32 || (aligned16(x) && aligned16(gate_w) && aligned16(up_w) && aligned16(act) && aligned16(saved)),
                 FMOE_ERR_ALIGNMENT, "%s: tensor pointers must be 16-byte aligned", who);
    hipStream_t s = (hipStream_t)stream;
    const int M = (int)num_tokens;
    switch (dtype) {
        case FMOE_F32: return gate_up_tiled<float>(x, gate_w, up_w, M, hidden, intermediate, act, saved, s);
        case FMOE_BF16: return gate_up_tiled<bf16_t>(x, gate_w, up_w, M, hidden, intermediate, act, saved, s);
        default: return gate_up_tiled<f16_t>(x, gate_w, up_w, M, hidden, intermediate, act, saved, s);
    }
}
}  // namespace
}  // namespace fmoe

extern "C" int fmoe_mlp_gate_up(const void* x, const void* gate_w, const void* up_w, int64_t num_tokens, int hidden,
                                int intermediate, int dtype, void* act, void* stream) {
    return fmoe::mlp_gate_up_impl("fmoe_mlp_gate_up", x, gate_w, up_w, num_tokens, hidden, intermediate, dtype, act, nullptr, stream);
}

extern "C" int fmoe_mlp_gate_up_save(const void* x, const void* gate_w, const void* up_w, int64_t num_tokens, int hidden,
                                     int intermediate, int dtype, void* act, void* saved, void* stream) {
    using namespace fmoe;
    if (saved == nullptr && num_tokens > 0) {
        clear_error();
        set_error("fmoe_mlp_gate_up_save: null buffer for the gate and up products");
        return FMOE_ERR_NULL_POINTER;
    }
    return mlp_gate_up_impl("fmoe_mlp_gate_up_save", x, gate_w, up_w, num_tokens, hidden, intermediate, dtype, act, saved, stream);
}

extern "C" int fmoe_mlp_down(const void* act, const void* down_w, int64_t num_tokens, int hidden, int intermediate,
                             int dtype, const void* residual, void* out, void* stream) {
    using namespace fmoe;
    clear_error();
    if (int rc = check_mlp_shape("fmoe_mlp_down", num_tokens, hidden, intermediate, dtype)) return rc;
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(act && down_w && out, FMOE_ERR_NULL_POINTER, "fmoe_mlp_down: null tensor pointer");
    FMOE_REQUIRE(dtype == FMOE_F32 || (aligned16(act) && aligned16(down_w)), FMOE_ERR_ALIGNMENT,
                 "fmoe_mlp_down: tensor pointers must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int M = (int)num_tokens;
    switch (dtype) {
        case FMOE_F32: return down_tiled<float>(act, down_w, M, hidden, intermediate, residual, out, s);
        case FMOE_BF16: return down_tiled<bf16_t>(act, down_w, M, hidden, intermediate, residual, out, s);
        default: return down_tiled<f16_t>(act, down_w, M, hidden, intermediate, residual, out, s);
    }
}

extern "C" int fmoe_mlp_forward(const void* x, const void* gate_w, const void* up_w, const void* down_w,
                                int64_t num_tokens, int hidden, int intermediate, int dtype, const void* residual,
                                void* out, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fmoe;
    clear_error();
    if (int rc = check_mlp_shape("fmoe_mlp_forward", num_tokens, hidden, intermediate, dtype)) return rc;
    if (num_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(x && gate_w && up_w && down_w && out, FMOE_ERR_NULL_POINTER, "fmoe_mlp_forward: null tensor pointer");
    const size_t need = fmoe_mlp_workspace_bytes(num_tokens, hidden, intermediate, dtype);
    FMOE_REQUIRE(workspace && workspace_bytes >= need, FMOE_ERR_WORKSPACE,
                 "fmoe_mlp_forward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (int rc = fmoe_mlp_gate_up(x, gate_w, up_w, num_tokens, hidden, intermediate, dtype, workspace, stream)) return rc;
    return fmoe_mlp_down(workspace, down_w, num_tokens, hidden, intermediate, dtype, residual, out, stream);
}
