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
//   * B slice [BK][BN] is stored the same way, [BK/8][BN][8 bf16], which needs a transposition: a
//     thread loads 8 rows (k) of 4 columns (8 bytes each, lanes on consecutive columns), builds for
//     each column the four (k, k+1) words with byte permutes and stores 16 bytes per column.  Column n
//     of a k-group sits at position n ^ ((n / 8) % 8), which makes these stores conflict-free (lanes
//     write every fourth column) and keeps the reads conflict-free.
//   * Row m of k-group kq of A sits at position m ^ swz(kq) for the same reason (the lanes that
//     store the k-groups of one row are 4096 bytes apart).
// With EDGE the tile may hang over the M x N x K problem and rows need not be aligned: loads outside
// read as zero (element loads where a 16-byte / 8-byte piece is not whole or not aligned), and the
// epilogue skips elements outside.  Without it: M % BM == 0, N % BN == 0, K % BK == 0, rows of A 16-byte
// and rows of B 8-byte aligned (the emitter checks).  Large tiles use the second variant further down
// (tile_accumulate_bf16_direct: slices loaded straight into an LDS ring); this one serves 64x64 tiles.
#ifndef TIRAMISU_AMD_GEMM_MFMA_BF16_HIP_H
#define TIRAMISU_AMD_GEMM_MFMA_BF16_HIP_H
#include "gemm_mfma.hip.h"

namespace tgemm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2), aligned(4)));

template <int BM_, int BN_, int BK_, int WGM_, int WGN_, bool EDGE_ = false>
struct config_bf16 {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
    static constexpr bool EDGE = EDGE_;
    static constexpr int NT = 64 * WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int A_WORDS = (BK / 8) * BM * 4;    // 32-bit words per stage
    static constexpr int B_WORDS = (BK / 8) * BN * 4;
    static constexpr int STAGE_WORDS = A_WORDS + B_WORDS;
    static constexpr int LDS_BYTES = 2 * STAGE_WORDS * 4;
    static constexpr int NVA = BM * (BK / 8) / NT;       // 16-byte loads of A per thread and slice
    static constexpr int UNITS_B = (BK / 8) * (BN / 4);  // (8-row x 4-column) units of B per slice
    static constexpr int NVB = (UNITS_B + NT - 1) / NT;  // units per thread and slice
    static_assert(BM * (BK / 8) % NT == 0, "tile must split evenly over the threads");
    static_assert(BK % 16 == 0, "BK must be a multiple of 16");
};

template <class CFG>
__device__ __forceinline__ void tile_accumulate_bf16(accumulators<CFG> &acc, const uint16_t *__restrict__ A, long lda,
                                                     const uint16_t *__restrict__ B, long ldb, int M, int N, int K, int m0, int n0,
                                                     uint32_t *lds) {
    // whole 16-byte pieces of A / 8-byte pieces of B may be loaded as such
    const bool vec_a = !CFG::EDGE || ((lda % 8 == 0) && ((uintptr_t)A % 16 == 0));
    const bool vec_b = !CFG::EDGE || ((ldb % 4 == 0) && ((uintptr_t)B % 8 == 0));
    constexpr int TM = CFG::TM, TN = CFG::TN, BK = CFG::BK, BM = CFG::BM, BN = CFG::BN, NT = CFG::NT;
    constexpr int NVA = CFG::NVA, NVB = CFG::NVB;
    constexpr int Q = BK / 16;                      // MFMA steps (fragment sets) per slice
    static_assert(Q >= 2 && Q % 2 == 0, "the pipeline needs an even number of MFMA steps per slice");
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;

    u32x4 ra[NVA];
    u32x2 rb[NVB][8];
    // stage addresses are computed from `lds` (never selected between pointers) so that every
    // access stays an LDS instruction
    auto stage_a = [&](int stage) -> uint32_t * { return lds + stage * CFG::STAGE_WORDS; };
    auto stage_b = [&](int stage) -> uint32_t * { return lds + stage * CFG::STAGE_WORDS + CFG::A_WORDS; };
    // row m of k-group kq sits at position m ^ swz(kq): the lanes that store the k-groups of one row
    // (4096 bytes apart) then hit different 16-byte bank groups
    auto swz = [](int kq) -> int { return (BK / 8 >= 8) ? (kq & 7) : 2 * (kq & 3); };

    auto load_a = [&](int k0) {
#pragma unroll
        for (int v = 0; v < NVA; v++) {
            const int idx = t + NT * v, kq = idx % (BK / 8), m = idx / (BK / 8);
            const uint16_t *p = A + (long)(m0 + m) * lda + k0 + 8 * kq;
            if (!CFG::EDGE || (vec_a && m0 + m < M && k0 + 8 * kq + 7 < K)) {
                ra[v] = *reinterpret_cast<const u32x4 *>(p);
            } else {
                uint16_t e[8];
#pragma unroll
                for (int i = 0; i < 8; i++) e[i] = (m0 + m < M && k0 + 8 * kq + i < K) ? p[i] : (uint16_t)0;
                ra[v] = u32x4{e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16), e[4] | ((uint32_t)e[5] << 16), e[6] | ((uint32_t)e[7] << 16)};
            }
        }
    };
    auto col_pos = [](int n) -> int { return n ^ ((n >> 3) & 7); };
    auto load_b = [&](int k0) {
#pragma unroll
        for (int v = 0; v < NVB; v++) {
            const int idx = t + NT * v, n4 = idx % (BN / 4), kq = idx / (BN / 4);
            if (CFG::UNITS_B % NT == 0 || idx < CFG::UNITS_B) {
                const uint16_t *p = B + (long)(k0 + 8 * kq) * ldb + n0 + 4 * n4;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    if (!CFG::EDGE || (vec_b && k0 + 8 * kq + i < K && n0 + 4 * n4 + 3 < N)) {
                        rb[v][i] = *reinterpret_cast<const u32x2 *>(p + i * ldb);
                    } else {
                        uint16_t e[4];
#pragma unroll
                        for (int c = 0; c < 4; c++) e[c] = (k0 + 8 * kq + i < K && n0 + 4 * n4 + c < N) ? p[i * ldb + c] : (uint16_t)0;
                        rb[v][i] = u32x2{e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16)};
                    }
                }
            }
        }
    };
    auto store_a = [&](int stage) {
#pragma unroll
        for (int v = 0; v < NVA; v++) {
            const int idx = t + NT * v, kq = idx % (BK / 8), m = idx / (BK / 8);
            *reinterpret_cast<u32x4 *>(stage_a(stage) + (kq * BM + (m ^ swz(kq))) * 4) = ra[v];
        }
    };
    auto store_b = [&](int stage) {
#pragma unroll
        for (int v = 0; v < NVB; v++) {
            const int idx = t + NT * v, n4 = idx % (BN / 4), kq = idx / (BN / 4);
            if (CFG::UNITS_B % NT == 0 || idx < CFG::UNITS_B) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // word p of column c = (row 2p, row 2p+1) as (low, high) halves
                    u32x4 w;
#pragma unroll
                    for (int pp = 0; pp < 4; pp++)
                        w[pp] = __builtin_amdgcn_perm(rb[v][2 * pp + 1][c >> 1], rb[v][2 * pp][c >> 1],
                                                      (c & 1) ? 0x07060302u : 0x05040100u);
                    *reinterpret_cast<u32x4 *>(stage_b(stage) + (kq * BN + col_pos(4 * n4 + c)) * 4) = w;
                }
            }
        }
    };
    bf16x8 fa[2][TM], fb[2][TN];                    // fragments: one set in use, one in flight
    auto read_frags = [&](int stage, int s, int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int kq = 2 * s + h, m = wm * CFG::WM + i * 32 + l32;
            const u32x4 w = *reinterpret_cast<const u32x4 *>(stage_a(stage) + (kq * BM + (m ^ swz(kq))) * 4);
            fa[buf][i] = __builtin_bit_cast(bf16x8, w);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int kq = 2 * s + h, n = wn * CFG::WN + j * 32 + l32;
            const u32x4 w = *reinterpret_cast<const u32x4 *>(stage_b(stage) + (kq * BN + col_pos(n)) * 4);
            fb[buf][j] = __builtin_bit_cast(bf16x8, w);
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][i], fb[buf][j], acc.t[i][j], 0, 0, 0);
    };

    // Same schedule as the fp32 loop (gemm_mfma.hip.h): while the matrix cores work through the
    // Q fragment sets of one slice, the next slice (in registers since the previous iteration) is
    // stored into the other stage -- A during set 0, B during set 1 -- each followed by the global
    // loads of the slice after it; the barrier sits before the last set, whose matrix instructions
    // cover the first fragment reads of the next slice.  Memory instructions are dealt out between
    // the matrix instructions with scheduling groups.
    const int KT = CFG::EDGE ? (K + BK - 1) / BK : K / BK;
    load_a(0);
    load_b(0);
    store_a(0);
    store_b(0);
    if (KT > 1) {
        load_a(BK);
        load_b(BK);
    }
    __syncthreads();
    read_frags(0, 0, 0);

    constexpr int MFMAS = TM * TN;
    constexpr int FRAG_READS = TM + TN;             // LDS read instructions per set
    auto slice = [&](int kt, auto more_c, auto load_c) {
        constexpr bool MORE = decltype(more_c)::value, LOAD = decltype(load_c)::value;
        const int cur = kt & 1;
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int buf = q & 1;
            if (q == 0 && MORE) {
                store_a(cur ^ 1);
                if (LOAD) load_a((kt + 2) * BK);
            }
            if (q == (Q > 2 ? 1 : 0) && MORE) {
                store_b(cur ^ 1);
                if (LOAD) load_b((kt + 2) * BK);
            }
            if (q + 1 < Q) {
                read_frags(cur, q + 1, buf ^ 1);
            } else {
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                if (MORE) read_frags(cur ^ 1, 0, buf ^ 1);
            }
            multiply(buf);
            if (q + 1 < Q || MORE) {
#pragma unroll
                for (int i = 0; i < MFMAS; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (q + 1 < Q && MORE) {
                        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                        if (LOAD) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                    if (i < FRAG_READS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            }
        }
    };
    int kt = 0;
    for (; kt + 2 < KT; kt++) slice(kt, std::true_type(), std::true_type());
    if (kt + 1 < KT) { slice(kt, std::true_type(), std::false_type()); kt++; }
    if (kt < KT) slice(kt, std::false_type(), std::false_type());
}

// ---------------------------------------------------------------------------------------------
// Variant whose operand slices go from global memory straight into LDS (buffer_load ... lds, 16 bytes
// per lane: lane l of a wave-wide load writes LDS bytes [base + 16 l, base + 16 l + 16), the global
// address is the lane's own), through a ring of STAGES slices: no staging registers, no LDS store
// instructions, and STAGES-1 slices in flight.
//   * A slice [BM][BK] is kept row-major in 16-byte granules (8 k), granule kq of row m at position
//     kq ^ swzA(m); one 16-byte LDS read is a lane's MFMA operand.
//   * B slice [BK][BN] is kept row-major as it is in memory ([k][n], granule = 8 columns), granule g
//     of row k at position g ^ swzB(k).  The MFMA operand (8 consecutive k of one column) comes
//     from two transposing LDS reads (ds_read_b64_tr_b16): within 16 lanes, lane L receives element
//     L % 4 of the 8 bytes addressed by lanes L / 4, L / 4 + 4, L / 4 + 8, L / 4 + 12; so lane r of
//     the 16 addresses row k0 + r / 4, columns n0 + 4 (r % 4) .. + 3, and lane L ends up with
//     (k0 .. k0 + 3, column n0 + L).
//   * The swizzles keep the reads free of bank conflicts whether the LDS serves 128 bytes (8 lanes of
//     a 16-byte read, 16 of a transposing one) or 256 bytes per cycle: swzA spreads 8 and 16
//     consecutive rows, swzB (0, 4, 10, 14 for k % 4) the four rows of a transposing read, over
//     distinct 16-byte bank groups in both cases (measured: SQ_LDS_BANK_CONFLICT = 0).
// A call ends with a barrier (every wave is past its last read), so it may be repeated for a second
// pair of operands.  Rows of A and of B must be 16-byte aligned.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int STAGES_>
struct config_bf16_direct {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, STAGES = STAGES_;
    static constexpr bool EDGE = false;
    static constexpr int NW = WGM * WGN, NT = 64 * NW;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int GA = BK / 8, GB = BN / 8;          // 16-byte granules per row of the A / B slice
    static constexpr int A_BYTES = BM * BK * 2, B_BYTES = BK * BN * 2, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int LA = BM * GA / 64 / NW, LB = BK * GB / 64 / NW;   // wave-wide loads per wave and slice
    static_assert(BK == 32 || BK == 64, "slices of 32 or 64 k");
    static_assert(BM * GA % (64 * NW) == 0 && BK * GB % (64 * NW) == 0, "slices must split evenly over the waves");
    static_assert(GB >= 16 && (GB & (GB - 1)) == 0, "row of B: a power of two of 128 columns or more (the swizzle spans 16 granules)");
    static_assert(STAGES >= 2, "the ring needs two stages or more");
};

template <int N> __device__ __forceinline__ void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <class CFG>
__device__ __forceinline__ void tile_accumulate_bf16_direct(accumulators<CFG> &acc, const uint16_t *__restrict__ A, long lda,
                                                            const uint16_t *__restrict__ B, long ldb, int M, int N, int K, int m0,
                                                            int n0, uint32_t *lds) {
    constexpr int TM = CFG::TM, TN = CFG::TN, BK = CFG::BK, GA = CFG::GA, GB = CFG::GB, LA = CFG::LA, LB = CFG::LB, ST = CFG::STAGES;
    constexpr int Q = BK / 16;
    typedef __attribute__((address_space(3))) char lds_char;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;
    lds_char *const base = (lds_char *)lds;
    auto swzA = [](int m) -> int { return GA == 8 ? ((m ^ (m >> 3)) & 7) : (((m >> 2) & 1) | ((((m >> 1) ^ (m >> 3)) & 1) << 1)); };
    auto swzB = [](int k) -> int { return ((k & 1) << 2) | ((k & 2) ? 10 : 0); };   // 0, 4, 10, 14

    // The loads are buffer loads (base in a resource descriptor, 32-bit byte offset per lane, one
    // scalar offset per operand that advances by a slice): no 64-bit address arithmetic in the loop,
    // and an address past the operand reads as zero instead of faulting.
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void *)A, 0, (int)((((long)M - 1) * lda + K) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, (int)((((long)K - 1) * ldb + N) * 2), 0x00020000);
    int va[LA], vb[LB];                              // per-lane byte offsets of this wave's loads within a slice
#pragma unroll
    for (int v = 0; v < LA; v++) {
        const int g = (wave * LA + v) * 64 + lane, m = g / GA, kq = (g % GA) ^ swzA(m);
        va[v] = (int)(((long)(m0 + m) * lda + 8 * kq) * 2);
    }
#pragma unroll
    for (int v = 0; v < LB; v++) {
        const int g = (wave * LB + v) * 64 + lane, k = g / GB, n8 = (g % GB) ^ swzB(k);
        vb[v] = (int)(((long)k * ldb + n0 + 8 * n8) * 2);
    }
    int sa_off = 0, sb_off = 0;                      // byte offsets of the next slice to request
    const int sb_step = (int)((long)BK * ldb * 2);
    auto issue_one = [&](int stage, int v) {
        if (v < LA) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void *)(base + stage * CFG::STAGE_BYTES + (wave * LA + v) * 1024), 16,
                                                     va[v], sa_off, 0, 0);
        } else {
            const int u = v - LA;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void *)(base + stage * CFG::STAGE_BYTES + CFG::A_BYTES + (wave * LB + u) * 1024),
                                                     16, vb[u], sb_off, 0, 0);
        }
        if (v == LA + LB - 1) {
            sa_off += BK * 2;
            sb_off += sb_step;
        }
    };
    auto issue = [&](int stage) {
#pragma unroll
        for (int v = 0; v < LA + LB; v++) issue_one(stage, v);
    };

    // fragment addresses within a stage, per MFMA step s: A granule (row, 2 s + h); B: two reads of four k
    int offA[TM], offB[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) offA[i] = wm * CFG::WM + i * 32 + l32;                    // row
    const int r16 = lane & 15, grp = lane >> 4;                                             // lane of the 16, group
#pragma unroll
    for (int j = 0; j < TN; j++) offB[j] = wn * CFG::WN + j * 32 + 16 * (grp & 1) + 4 * (r16 & 3);   // first column addressed
    const int kB = 8 * (grp >> 1) + (r16 >> 2);                                            // row addressed within the step (first read)

    // fragments: one set in use, one in flight; B fragments arrive as two halves (four k each)
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    bf16x8 fa[2][TM];
    s16x4 fbl[2][TN], fbh[2][TN];
    constexpr int MFMAS = TM * TN, READS = TM + 2 * TN;
    // read number r of a step, in the order the matrix instructions need them (row 0 of A, all of B,
    // the other rows of A)
    auto read_one = [&](int stage, int s, int buf, int r) {
        lds_char *const sa = base + stage * CFG::STAGE_BYTES, *const sb = sa + CFG::A_BYTES;
        if (r == 0 || r > 2 * TN) {
            const int i = r == 0 ? 0 : r - 2 * TN;
            const int m = offA[i], kq = 2 * s + h;
            const u32x4 w = *reinterpret_cast<const __attribute__((address_space(3))) u32x4 *>(sa + (m * GA + (kq ^ swzA(m))) * 16);
            fa[buf][i] = __builtin_bit_cast(bf16x8, w);
        } else {
            const int j = (r - 1) / 2, half = (r - 1) % 2;
            const int k = 16 * s + kB + 4 * half, n = offB[j];
            const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(sb + (k * GB + ((n >> 3) ^ swzB(k))) * 16 + (n & 7) * 2));
            if (half) fbh[buf][j] = v; else fbl[buf][j] = v;
        }
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / TN, j = idx % TN;
        const s16x8 both = __builtin_shufflevector(fbl[buf][j], fbh[buf][j], 0, 1, 2, 3, 4, 5, 6, 7);
        acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][i], __builtin_bit_cast(bf16x8, both), acc.t[i][j], 0, 0, 0);
    };

    // Ring: slice kt lives in stage kt % STAGES; all stages are requested up front.  In the last MFMA
    // step of slice kt, after its first PRE matrix instructions (the wave's last reads of the slice,
    // issued a dozen matrix instructions earlier, have returned by then), one barrier both publishes
    // slice kt+1 (every wave waited for its own loads of it) and retires slice kt's stage, into which
    // slice kt+STAGES is requested: STAGES-1 slices of matrix work cover a load.  The instruction
    // order is pinned (a scheduling barrier after every matrix instruction): the LDS reads of the next
    // step's fragments -- and, after the barrier, the slice's loads -- are dealt out behind the matrix
    // instructions, with large wave tiles one read each, so that a fragment is requested at least seven
    // matrix instructions before its use and the compiler's waits count exactly (buffer loads, unlike
    // global or flat ones, do not make it wait for every outstanding LDS access).
    const int KT = K / BK;
    constexpr int PER = LA + LB;                    // loads per wave and slice
    constexpr int PRE = MFMAS >= 16 ? 4 : 1;        // matrix instructions of the last step ahead of the barrier
    static_assert((ST - 1) * PER <= 63, "the load counter holds 63");
    constexpr int SLOTS = READS < MFMAS ? (READS > MFMAS - 4 ? READS : MFMAS - 4) : MFMAS;   // matrix instructions of a step that are followed by reads
#pragma unroll
    for (int p = 0; p < ST; p++)
        if (p < KT) issue(p);
    if (KT >= ST) wait_vmcnt<(ST - 1) * PER>(); else wait_vmcnt<0>();      // slice 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < READS; r++) read_one(0, 0, 0, r);
    // ISSUE: slice kt+STAGES exists (steady state: exactly STAGES-2 requests are behind slice kt+1);
    // MORE: slice kt+1 exists
    auto slice = [&](int stage, int next, auto issue_c, auto more_c) {
        constexpr bool ISSUE = decltype(issue_c)::value, MORE = decltype(more_c)::value;
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int buf = q & 1;
            if (q + 1 < Q) {
#pragma unroll
                for (int idx = 0; idx < MFMAS; idx++) {
                    mfma_one(buf, idx);
#pragma unroll
                    for (int r = idx * READS / SLOTS; r < (idx + 1) * READS / SLOTS; r++) read_one(stage, q + 1, buf ^ 1, r);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else if (MORE) {
#pragma unroll
                for (int idx = 0; idx < PRE; idx++) {
                    mfma_one(buf, idx);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (ISSUE) wait_vmcnt<(ST - 2) * PER>(); else wait_vmcnt<0>();
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int idx = PRE; idx < MFMAS; idx++) {
                    mfma_one(buf, idx);
#pragma unroll
                    for (int r = (idx - PRE) * READS / (MFMAS - PRE); r < (idx - PRE + 1) * READS / (MFMAS - PRE); r++) read_one(next, 0, buf ^ 1, r);
                    if (ISSUE) {
#pragma unroll
                        for (int v = (idx - PRE) * PER / (MFMAS - PRE); v < (idx - PRE + 1) * PER / (MFMAS - PRE); v++) issue_one(stage, v);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int idx = 0; idx < MFMAS; idx++) mfma_one(buf, idx);
            }
        }
    };
    int kt = 0, stage = 0;
    auto advance = [&]() { kt++; stage = stage + 1 == ST ? 0 : stage + 1; };
    for (; kt + ST < KT; advance()) slice(stage, stage + 1 == ST ? 0 : stage + 1, std::true_type(), std::true_type());
    for (; kt + 1 < KT; advance()) slice(stage, stage + 1 == ST ? 0 : stage + 1, std::false_type(), std::true_type());
    if (kt < KT) slice(stage, 0, std::false_type(), std::false_type());
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

}  // namespace tgemm
#endif
