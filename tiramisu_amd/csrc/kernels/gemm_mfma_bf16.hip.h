// bf16-input / fp32-accumulate dense contraction on the gfx950 matrix cores
// (v_mfma_f32_32x32x16_bf16): C[m,n] = epilogue(sum_k A[m,k] * B[k,n]) with A row-major
// (K contiguous) and B row-major (N contiguous), both stored as bf16, C in fp32.
//
// Same workgroup structure as the fp32 kernel (gemm_mfma.hip.h): WGM x WGN wave64 wavefronts, each
// owning 32x32 accumulator tiles; two LDS stages, one barrier per K-slice, global->register
// prefetch of the next slice.  One MFMA consumes 16 k: a lane holds 8 consecutive k of its row
// (A) or column (B); lanes 0-31 take k = 0..7 of the step, lanes 32-63 take k = 8..15.
//   * A slice [BM][BK] is stored as [BK/8][BM][8 bf16]: a 16-byte global load is a 16-byte LDS
//     store, and one 16-byte LDS read is a lane's whole MFMA operand.
//   * B slice [BK][BN] is stored as k-pairs, [BK/2][BN][2 bf16]: a thread loads two rows of 8
//     columns, interleaves them in registers (one 32-bit word per (k pair, n)) and stores 32
//     bytes; a lane assembles its operand from four conflict-free 4-byte reads (lanes read
//     consecutive words).
// Whole tiles only: M % BM == 0, N % BN == 0, K % BK == 0, rows 16-byte aligned (the emitter checks).
#ifndef TIRAMISU_AMD_GEMM_MFMA_BF16_HIP_H
#define TIRAMISU_AMD_GEMM_MFMA_BF16_HIP_H
#include "gemm_mfma.hip.h"

namespace tgemm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int BM_, int BN_, int BK_, int WGM_, int WGN_>
struct config_bf16 {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
    static constexpr bool EDGE = false;
    static constexpr int NT = 64 * WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int A_WORDS = (BK / 8) * BM * 4;    // 32-bit words per stage
    static constexpr int B_WORDS = (BK / 2) * BN;
    static constexpr int STAGE_WORDS = A_WORDS + B_WORDS;
    static constexpr int LDS_BYTES = 2 * STAGE_WORDS * 4;
    static constexpr int NVA = BM * (BK / 8) / NT;       // 16-byte loads of A per thread and slice
    static constexpr int NVB = (BK / 2) * (BN / 8) / NT; // (two-row x 8-column) units of B per thread and slice
    static_assert(BM * (BK / 8) % NT == 0 && (BK / 2) * (BN / 8) % NT == 0, "tile must split evenly over the threads");
    static_assert(BK % 16 == 0, "BK must be a multiple of 16");
};

template <class CFG>
__device__ __forceinline__ void tile_accumulate_bf16(accumulators<CFG> &acc, const uint16_t *__restrict__ A, long lda,
                                                     const uint16_t *__restrict__ B, long ldb, int K, int m0, int n0,
                                                     uint32_t *lds) {
    constexpr int TM = CFG::TM, TN = CFG::TN, BK = CFG::BK, BM = CFG::BM, BN = CFG::BN, NT = CFG::NT;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;

    u32x4 ra[CFG::NVA], rb0[CFG::NVB], rb1[CFG::NVB];
    uint32_t *sA[2] = {lds, lds + CFG::STAGE_WORDS};
    uint32_t *sB[2] = {lds + CFG::A_WORDS, lds + CFG::STAGE_WORDS + CFG::A_WORDS};

    auto load = [&](int k0) {
#pragma unroll
        for (int v = 0; v < CFG::NVA; v++) {
            const int idx = t + NT * v, kq = idx % (BK / 8), m = idx / (BK / 8);
            ra[v] = *reinterpret_cast<const u32x4 *>(A + (long)(m0 + m) * lda + k0 + 8 * kq);
        }
#pragma unroll
        for (int v = 0; v < CFG::NVB; v++) {
            const int idx = t + NT * v, n8 = idx % (BN / 8), kp = idx / (BN / 8);
            const uint16_t *p = B + (long)(k0 + 2 * kp) * ldb + n0 + 8 * n8;
            rb0[v] = *reinterpret_cast<const u32x4 *>(p);
            rb1[v] = *reinterpret_cast<const u32x4 *>(p + ldb);
        }
    };
    auto store = [&](int stage) {
#pragma unroll
        for (int v = 0; v < CFG::NVA; v++) {
            const int idx = t + NT * v, kq = idx % (BK / 8), m = idx / (BK / 8);
            *reinterpret_cast<u32x4 *>(sA[stage] + (kq * BM + m) * 4) = ra[v];
        }
#pragma unroll
        for (int v = 0; v < CFG::NVB; v++) {
            const int idx = t + NT * v, n8 = idx % (BN / 8), kp = idx / (BN / 8);
            // word j of the output = (row0[j], row1[j]) as (low, high) halves
            u32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t a = rb0[v][i], b = rb1[v][i];
                const uint32_t even = (a & 0xffffu) | (b << 16), odd = (a >> 16) | (b & 0xffff0000u);
                if (i < 2) { lo[2 * i] = even; lo[2 * i + 1] = odd; }
                else       { hi[2 * (i - 2)] = even; hi[2 * (i - 2) + 1] = odd; }
            }
            uint32_t *q = sB[stage] + kp * BN + 8 * n8;
            *reinterpret_cast<u32x4 *>(q) = lo;
            *reinterpret_cast<u32x4 *>(q + 4) = hi;
        }
    };

    const int KT = K / BK;
    load(0);
    store(0);
    __syncthreads();
    for (int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) load((kt + 1) * BK);
#pragma unroll
        for (int s = 0; s < BK / 16; s++) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(sA[cur] + ((2 * s + h) * BM + wm * CFG::WM + i * 32 + l32) * 4);
                fa[i] = __builtin_bit_cast(bf16x8, w);
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const uint32_t *p = sB[cur] + (8 * s + 4 * h) * BN + wn * CFG::WN + j * 32 + l32;
                const u32x4 w = {p[0], p[BN], p[2 * BN], p[3 * BN]};
                fb[j] = __builtin_bit_cast(bf16x8, w);
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc.t[i][j], 0, 0, 0);
        }
        if (more) store(cur ^ 1);
        __syncthreads();
    }
}

}  // namespace tgemm
#endif
