// fp64 GEMM on the matrix cores of gfx950 (v_mfma_f64_16x16x4_f64): C = alpha * op(A) * op(B) + beta * C with
// every operand addressed through two strides, so that one kernel serves all four transposition cases of the
// library call, leading dimensions and offsets included.
//
// A workgroup of WGM x WGN wavefronts computes a tile of (16 TM WGM) x (16 TN WGN) elements, TM x TN instruction
// tiles of 16 x 16 per wavefront (128 x 128 on 2 x 4 wavefronts of 4 x 2 instruction tiles: two wavefronts per
// SIMD cover each other's waits; 64 x 64 on 2 x 2 wavefronts for problems that would not fill the chip with the
// large tile).  K is walked in slices of 16: the slice's A and B parts go from
// global memory to registers (8-byte loads, the thread-to-element mapping chosen so that consecutive lanes follow
// the operand's unit stride), from there to one of two LDS stages as [k][m] and [k][n] (rows padded so that the
// 16 lanes of an instruction operand read 16 consecutive doubles), and each of the 4 k-steps of a slice reads
// TM + TN operand fragments for TM * TN matrix instructions.  The next slice's global loads are issued before the
// current slice is multiplied and stored to the other stage after it: one barrier per slice.
// Loads outside the operands give zeros and the epilogue skips what lies outside C, so any M, N, K is accepted.
//
// Instruction layout (one wavefront): lane l supplies A[row l % 16][k l / 16] and B[k l / 16][column l % 16];
// its four results are rows l / 16 + 0, 4, 8, 12 of column l % 16.
#ifndef TIRAMISU_AMD_GEMM_MFMA_F64_HIP_H
#define TIRAMISU_AMD_GEMM_MFMA_F64_HIP_H
#include <hip/hip_runtime.h>

#include "gemm_mfma.hip.h"

namespace tgemm64 {

typedef double f64x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 16;

template <int TM_, int TN_, int WGM_, int WGN_, int PAD = 4>
struct shape {
    static constexpr int TM = TM_, TN = TN_, WGM = WGM_, WGN = WGN_;
    static constexpr int NT = 64 * WGM * WGN;
    static constexpr int BM = 16 * TM * WGM, BN = 16 * TN * WGN;
    static constexpr int A_ROW = BM + PAD, B_ROW = BN + PAD;                 // doubles per k row of a stage
    static constexpr int STAGE = BK * (A_ROW + B_ROW);
    static constexpr int LDS_BYTES = 2 * STAGE * (int)sizeof(double);
    static constexpr int A_PER_THREAD = BM * BK / NT, B_PER_THREAD = BN * BK / NT;   // elements per thread and slice
    static_assert((BM * BK) % NT == 0 && (BN * BK) % NT == 0, "slice parts divide over the threads");
};

// The second launch bound (wavefronts per SIMD) holds the kernel to the registers that let two workgroups share a
// compute unit: at 136 registers instead of 128 a single workgroup is resident and the kernel is a quarter slower.
// A_KFAST: consecutive k of A are adjacent in memory (stride_ak == 1), else consecutive m are; likewise B_NFAST.
template <class S, bool A_KFAST, bool B_NFAST>
__global__ void __launch_bounds__(S::NT, S::NT / 128) dgemm_kernel(const double *__restrict__ A, const double *__restrict__ B, double *__restrict__ C, int M, int N,
                                                   int K, long stride_am, long stride_ak, long stride_bk, long stride_bn, long ldc, double alpha,
                                                   double beta) {
    constexpr int TM = S::TM, TN = S::TN, NT = S::NT;
    extern __shared__ __attribute__((aligned(16))) double lds64[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave / S::WGN, wn = wave % S::WGN;
    const int l16 = lane & 15, kq = lane >> 4;
    // the workgroups of one XCD (ids congruent modulo 8) cover a compact group of C tiles: the panels of A and B
    // that they share are fetched once into that XCD's L2
    int tile_m, tile_n;
    tgemm::tile_of_block((M + S::BM - 1) / S::BM, (N + S::BN - 1) / S::BN, tile_m, tile_n);
    const int m0 = tile_m * S::BM, n0 = tile_n * S::BN;

    double ra[S::A_PER_THREAD], rb[S::B_PER_THREAD];
    auto load_slice = [&](int k0) {
#pragma unroll
        for (int v = 0; v < S::A_PER_THREAD; v++) {
            const int u = t + NT * v;
            const int am = A_KFAST ? u / BK : u % S::BM, ak = A_KFAST ? u % BK : u / S::BM;
            const bool a_in = m0 + am < M && k0 + ak < K;
            const double a = A[a_in ? (long)(m0 + am) * stride_am + (long)(k0 + ak) * stride_ak : 0L];
            ra[v] = a_in ? a : 0.0;
        }
#pragma unroll
        for (int v = 0; v < S::B_PER_THREAD; v++) {
            const int u = t + NT * v;
            const int bn = B_NFAST ? u % S::BN : u / BK, bk = B_NFAST ? u / S::BN : u % BK;
            const bool b_in = n0 + bn < N && k0 + bk < K;
            const double b = B[b_in ? (long)(k0 + bk) * stride_bk + (long)(n0 + bn) * stride_bn : 0L];
            rb[v] = b_in ? b : 0.0;
        }
    };
    auto store_slice = [&](int stage) {
        double *la = lds64 + stage * S::STAGE, *lb = la + BK * S::A_ROW;
#pragma unroll
        for (int v = 0; v < S::A_PER_THREAD; v++) {
            const int u = t + NT * v;
            const int am = A_KFAST ? u / BK : u % S::BM, ak = A_KFAST ? u % BK : u / S::BM;
            la[ak * S::A_ROW + am] = ra[v];
        }
#pragma unroll
        for (int v = 0; v < S::B_PER_THREAD; v++) {
            const int u = t + NT * v;
            const int bn = B_NFAST ? u % S::BN : u / BK, bk = B_NFAST ? u / S::BN : u % BK;
            lb[bk * S::B_ROW + bn] = rb[v];
        }
    };

    f64x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

    const int slices = (K + BK - 1) / BK;
    if (slices > 0) {
        load_slice(0);
        store_slice(0);
    }
    __syncthreads();
    for (int s = 0; s < slices; s++) {
        const int stage = s & 1;
        if (s + 1 < slices) load_slice((s + 1) * BK);
        const double *la = lds64 + stage * S::STAGE + wm * (16 * TM) + l16;
        const double *lb = lds64 + stage * S::STAGE + BK * S::A_ROW + wn * (16 * TN) + l16;
#pragma unroll
        for (int ks = 0; ks < BK / 4; ks++) {
            double fa[TM], fb[TN];
            const int k = 4 * ks + kq;
#pragma unroll
            for (int i = 0; i < TM; i++) fa[i] = la[k * S::A_ROW + 16 * i];
#pragma unroll
            for (int j = 0; j < TN; j++) fb[j] = lb[k * S::B_ROW + 16 * j];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < slices) store_slice(stage ^ 1);
        __syncthreads();
    }

    // epilogue: the values of a row of instruction tiles first (they read C when beta != 0), then their stores
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int pass = 0; pass < 2; pass++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int row = m0 + wm * (16 * TM) + 16 * i + 4 * r + kq, col = n0 + wn * (16 * TN) + 16 * j + l16;
                    if (row < M && col < N) {
                        double *p = C + (long)row * ldc + col;
                        if (pass == 0) acc[i][j][r] = beta == 0.0 ? alpha * acc[i][j][r] : alpha * acc[i][j][r] + beta * *p;
                        else *p = acc[i][j][r];
                    }
                }
    }
}

}  // namespace tgemm64
#endif
