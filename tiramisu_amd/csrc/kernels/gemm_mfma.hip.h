// fp32 dense contraction on the gfx950 matrix cores: C[m,n] = epilogue(sum_k A[m,k] * B[k,n]).
//
// One workgroup of WGM x WGN wave64 wavefronts computes a BM x BN tile of C; each wavefront
// owns (BM/WGM) x (BN/WGN) of it as 32x32 accumulator tiles of v_mfma_f32_32x32x2_f32
// (16 accumulator registers per tile and lane).  K is walked in slices of BK through two
// LDS stages: while the matrix cores work on one stage, the next slice travels
// global -> registers -> other stage, with a single workgroup barrier per slice.
//
// LDS layouts are chosen so that neither the global loads nor the LDS accesses need a
// transposition in registers:
//   * an operand whose K index is contiguous in memory (row-major A, or a transposed B) is
//     stored K-interleaved, [BK/4][X+PAD][4]: a 16-byte global load is a 16-byte LDS store, and a
//     lane fetches 4 consecutive k for its row with one 16-byte LDS read (one read feeds 4 MFMA).
//     Row x of k-group kq sits at position x ^ 2*(kq % 4): the 8 lanes that store one 128-byte
//     piece of two rows then hit 8 different 16-byte bank groups instead of 2;
//   * an operand whose M/N index is contiguous (row-major B, or a transposed A) is stored as
//     it lies, [BK][X]: 16-byte stores, 4-byte conflict-free reads (lanes read consecutive words).
// For one 16-byte read q, the lower half of the wave (lanes 0-31) holds k = 8q+0..3 and the
// upper half k = 8q+4..7; MFMA step s multiplies the pairs {8q+s, 8q+4+s} -- both operands use
// the same assignment, which is all the instruction requires.
//
// The block index is remapped so that the workgroups that run on one XCD (hardware deals
// consecutive workgroup ids round-robin over the 8 XCDs) cover a compact group of C tiles and
// share their A rows / B columns in that XCD's L2.
#ifndef TIRAMISU_AMD_GEMM_MFMA_HIP_H
#define TIRAMISU_AMD_GEMM_MFMA_HIP_H
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "target_gfx950.h"

namespace tgemm {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));   // 4-byte aligned 16-byte load

// Data handed from one workgroup to another within a launch (partial tiles of a reduction cut over workgroups):
// written through to memory and read from there, as agent-scope atomic accesses of 8 bytes.  The compute dies of
// the GPU have an L2 cache each, so ordinary stores would need the writer's whole L2 written back (what an
// agent-scope release fence does) and the reader's invalidated; with these accesses the writer only has to wait
// for its own stores (handed_over_stores_done) before it announces them with an atomic counter, and the reader,
// once it has seen the counter, reads what the writers wrote.
__device__ __forceinline__ void store_handed_over(f32x4 *p, f32x4 v) {
    typedef unsigned long long u64;
    union { f32x4 v; u64 u[2]; } x;
    x.v = v;
    __hip_atomic_store(reinterpret_cast<u64 *>(p), x.u[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(reinterpret_cast<u64 *>(p) + 1, x.u[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 load_handed_over(const f32x4 *p) {
    typedef unsigned long long u64;
    union { f32x4 v; u64 u[2]; } x;
    u64 *q = reinterpret_cast<u64 *>(const_cast<f32x4 *>(p));
    x.u[0] = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    x.u[1] = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return x.v;
}
// every store_handed_over of this wavefront has reached memory when this returns.  The wait is written out: a
// release fence at workgroup scope orders the stores for the wavefronts of this compute unit only and, outside
// thread-group-split mode, waits for nothing (a reader on another die then sees the counter before the data).
// This relies on what gfx942 / gfx950 do, not on the HIP memory model: an agent-scope relaxed atomic store is
// written through to memory (sc1), vmcnt counts it down when memory has acknowledged it, and 0x0F70 is the gfx9
// encoding of "vmcnt(0) only".  Any other target takes the portable form: an agent-scope release fence (which
// writes the whole L2 back: correct, slow); TIRAMISU_PORTABLE_HANDOVER forces it here too.
__device__ __forceinline__ void handed_over_stores_done() {
#if (defined(__gfx950__) || defined(__gfx942__)) && !defined(TIRAMISU_PORTABLE_HANDOVER)
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0), leaving expcnt and lgkmcnt alone
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
#elif defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#endif
}
// no load_handed_over is moved ahead of this point (placed behind the counter's read)
__device__ __forceinline__ void handed_over_loads_begin() {
#if (defined(__gfx950__) || defined(__gfx942__)) && !defined(TIRAMISU_PORTABLE_HANDOVER)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#else
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
}

// An operand stored with one unit stride: element (x, k) lives at base[x*ld + k] (KMAJOR) or
// base[k*ld + x].  With EDGE, elements outside XE x KE read as zero and rows need not be
// 16-byte aligned (vec_ok false).
template <bool KMAJOR, bool EDGE>
struct linear_source {
    const float *__restrict__ base;
    long ld;
    int XE, KE;
    bool vec_ok;
    __device__ __forceinline__ f32x4 load4(int x, int k) const {
        const long off = KMAJOR ? (long)x * ld + k : (long)k * ld + x;
        if (!EDGE) return *reinterpret_cast<const f32x4 *>(base + off);
        const bool full = KMAJOR ? (x < XE && k + 3 < KE) : (k < KE && x + 3 < XE);
        if (full && vec_ok) return *reinterpret_cast<const f32x4 *>(base + off);
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int xx = KMAJOR ? x : x + e, kk = KMAJOR ? k + e : k;
            if (xx < XE && kk < KE) r[e] = base[KMAJOR ? (long)xx * ld + kk : (long)kk * ld + xx];
        }
        return r;
    }
};

// Columns of C (rows x of the B operand) dealt to tiles in groups: the operand's XE-long x range is
// made of column groups that lie UE apart (x = q * UE + u), and a tile of BN columns takes UB = BN / G
// consecutive units u out of every one of the G groups -- tile position x' stands for
//     x = (x' % BN / UB) * UE + (x' / BN) * UB + x' % UB.
// A workgroup then owns all G columns of its units, which is what an epilogue that combines them
// (the gates of a recurrent cell) needs.  UB must be a multiple of 4 for operands whose x is contiguous.
template <int BN, int UB>
__device__ __forceinline__ int regrouped_index(int x, int UE) {
    return ((x % BN) / UB) * UE + (x / BN) * UB + (x % UB);
}
template <class SRC, int BN, int UB>
struct regrouped_rows {
    SRC src;
    int UE;
    __device__ __forceinline__ auto load4(int x, int k) const { return src.load4(regrouped_index<BN, UB>(x, UE), k); }
};

// Two operands behind one another along k: k < K1 reads the first, the rest the second (from its own
// k = 0).  Lets several product terms that feed the same accumulators run as one pipelined loop;
// K1 must be a multiple of 4 (a 16-byte load along k never straddles the seam).
template <class S1, class S2>
struct concat_k {
    S1 first;
    S2 second;
    int K1;
    __device__ __forceinline__ f32x4 load4(int x, int k) const { return k < K1 ? first.load4(x, k) : second.load4(x, k - K1); }
};

// One operand tile of X x BK elements (X = BM for A, BN for B).
template <int X, int BK, int NT, bool KMAJOR, bool EDGE, int PAD>
struct operand_tile {
    static constexpr int UNITS = X * BK / 4;                      // 16-byte loads per slice
    static constexpr int NV = (UNITS + NT - 1) / NT;              // ... per thread (the last round may be partial)
    static constexpr bool PARTIAL = UNITS % NT != 0;
    static constexpr int ROW = KMAJOR ? (X + PAD) * 4 : X;      // LDS floats per k-group / per k
    static constexpr int LDS_FLOATS = KMAJOR ? (BK / 4) * ROW : BK * ROW;
    static_assert(BK % 8 == 0, "BK must be a multiple of 8");

    static __device__ __forceinline__ int swizzle(int x, int kq) { return x ^ (2 * (kq & 3)); }

    // SRC::load4(x, k) returns 4 consecutive elements along the operand's contiguous direction:
    // (x, k..k+3) for a K-major operand, (x..x+3, k) otherwise.
    template <class SRC>
    static __device__ __forceinline__ void load_global(const SRC &src, int x0, int k0, f32x4 (&regs)[NV]) {
        const int t = threadIdx.x;
#pragma unroll
        for (int v = 0; v < NV; v++) {
            const int idx = t + NT * v;
            if (PARTIAL && idx >= UNITS) break;
            int x, k;
            if (KMAJOR) { k = 4 * (idx % (BK / 4)); x = idx / (BK / 4); }
            else        { x = 4 * (idx % (X / 4));  k = idx / (X / 4); }
            regs[v] = src.load4(x0 + x, k0 + k);
        }
    }

    static __device__ __forceinline__ void store_lds(float *lds, const f32x4 (&regs)[NV]) {
        const int t = threadIdx.x;
#pragma unroll
        for (int v = 0; v < NV; v++) {
            const int idx = t + NT * v;
            if (PARTIAL && idx >= UNITS) break;
            if (KMAJOR) {
                const int kq = idx % (BK / 4), x = idx / (BK / 4);
                *reinterpret_cast<f32x4 *>(lds + kq * ROW + swizzle(x, kq) * 4) = regs[v];
            } else {
                const int xq = idx % (X / 4), k = idx / (X / 4);
                *reinterpret_cast<f32x4 *>(lds + k * ROW + 4 * xq) = regs[v];
            }
        }
    }

    // Values for the 4 MFMA steps of 16-byte read q: out[s] = element (x, 8q + 4h + s).
    static __device__ __forceinline__ f32x4 read_frag(const float *lds, int x, int q, int h) {
        if (KMAJOR) {
            return *reinterpret_cast<const f32x4 *>(lds + (2 * q + h) * ROW + swizzle(x, 2 * q + h) * 4);
        } else {
            const float *p = lds + (8 * q + 4 * h) * ROW + x;
            f32x4 r = {p[0], p[ROW], p[2 * ROW], p[3 * ROW]};
            return r;
        }
    }
};

// Position of the workgroup's tile: consecutive ids on one XCD walk groups of GROUP tile-rows.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    int id = blockIdx.x;
    constexpr int XCDS = ttarget::XCDS;
    if (total % XCDS == 0) id = (id % XCDS) * (total / XCDS) + id / XCDS;
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int g = id / per_group;
    const int first_m = g * GROUP;
    const int gsize = (tiles_m - first_m < GROUP) ? (tiles_m - first_m) : GROUP;
    tm = first_m + (id % per_group) % gsize;
    tn = (id % per_group) / gsize;
}

// WGM x WGN wavefronts tile the block in M and N; WGK > 1 adds groups of wavefronts that each take
// 1/WGK of every K-slice for the same C tile (for problems with too few C tiles to fill the chip);
// their partial sums are added through LDS by tile_reduce_k before the epilogue.
// DEPTH is the number of K-slices a thread keeps in flight in registers (1: the next slice only);
// latency-bound problems (few, short slices per workgroup) ask for all their slices at once.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, bool A_KMAJOR_, bool B_KMAJOR_, bool EDGE_, int PAD_ = 1, int WGK_ = 1,
          int DEPTH_ = 1>
struct config {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, WGK = WGK_, DEPTH = DEPTH_;
    static constexpr bool A_KMAJOR = A_KMAJOR_, B_KMAJOR = B_KMAJOR_, EDGE = EDGE_;
    static constexpr int NT = 64 * WGM * WGN * WGK;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    typedef operand_tile<BM, BK, NT, A_KMAJOR, EDGE, PAD_> opA;
    typedef operand_tile<BN, BK, NT, B_KMAJOR, EDGE, PAD_> opB;
    static constexpr int STAGE_FLOATS = opA::LDS_FLOATS + opB::LDS_FLOATS;
    static constexpr int LDS_BYTES = 2 * STAGE_FLOATS * 4;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32 MFMA tiles");
    static_assert((BK / 8) % WGK == 0, "the K-slice must split evenly over the K groups");
    static_assert(WGK == 1 || (WGK - 1) * WGM * WGN * TM * TN * 16 * 64 <= 2 * STAGE_FLOATS, "LDS too small for the K reduction");
};

// Accumulator tiles of one wavefront.
template <class CFG>
struct accumulators {
    f32x16 t[CFG::TM][CFG::TN];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int i = 0; i < CFG::TM; i++)
#pragma unroll
            for (int j = 0; j < CFG::TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) t[i][j][r] = 0.f;
    }
};

// acc += A(m0.., :) * B(:, n0..) over K, the operands read through sources (linear_source, or
// an emitter-generated gather such as the im2col view of a convolution input).  `lds` must hold
// config::LDS_BYTES bytes; all threads of the workgroup must call this together (it ends with a
// barrier, so it may be called again, e.g. for a second pair of operands feeding the same
// accumulators).
template <class CFG, class SRCA, class SRCB>
__device__ __forceinline__ void tile_accumulate(accumulators<CFG> &acc, const SRCA &A, const SRCB &B, int K, int m0,
                                                int n0, float *lds) {
    typedef typename CFG::opA opA;
    typedef typename CFG::opB opB;
    constexpr int TM = CFG::TM, TN = CFG::TN, BK = CFG::BK;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wk = wave / (CFG::WGM * CFG::WGN), wmn = wave % (CFG::WGM * CFG::WGN);
    const int wm = wmn / CFG::WGN, wn = wmn % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;

    constexpr int D = CFG::DEPTH;
    f32x4 ra[D][opA::NV], rb[D][opB::NV];           // slice s travels in slot s % D
    // stage addresses are computed from `lds` (never selected between pointers) so that every
    // access stays an LDS instruction
    auto stage_a = [&](int stage) -> float * { return lds + stage * CFG::STAGE_FLOATS; };
    auto stage_b = [&](int stage) -> float * { return lds + stage * CFG::STAGE_FLOATS + opA::LDS_FLOATS; };
    constexpr int Q = BK / 8 / CFG::WGK;            // 16-byte fragment reads per slice (of this wavefront's K group)
    static_assert(Q >= 2 && Q % 2 == 0, "the pipeline needs an even number of fragment reads per slice");
    f32x4 fa[2][TM], fb[2][TN];                     // fragments: one set in use, one in flight

    auto read_frags = [&](int stage, int q, int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++) fa[buf][i] = opA::read_frag(stage_a(stage), wm * CFG::WM + i * 32 + l32, wk * Q + q, h);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[buf][j] = opB::read_frag(stage_b(stage), wn * CFG::WN + j * 32 + l32, wk * Q + q, h);
    };

    // Schedule of one slice (stage `cur` holds it, its first fragments are already in registers):
    //   q = 0       store the next slice (in registers since the previous iteration) into the other
    //               stage, ask global memory for the slice after it, read fragments q+1, multiply;
    //   ...
    //   q = Q-1     barrier (the other stage is complete; every fragment of this stage was read
    //               before it), read the first fragments of the next slice, multiply.
    // So the LDS store, the barrier and the first LDS reads of a slice are all covered by matrix
    // instructions of the previous one, with a single barrier per slice.  Within a block of matrix
    // instructions the memory instructions are dealt out one per matrix instruction (scheduling
    // group barriers below); the steady-state slice is branch-free so that this is one scheduling
    // region, and the last two slices are peeled.
    const int KT = (K + BK - 1) / BK;
    opA::load_global(A, m0, 0, ra[0]);
    opB::load_global(B, n0, 0, rb[0]);
    opA::store_lds(stage_a(0), ra[0]);
    opB::store_lds(stage_b(0), rb[0]);
#pragma unroll
    for (int s = 1; s <= D; s++)
        if (s < KT) {
            opA::load_global(A, m0, s * BK, ra[s % D]);
            opB::load_global(B, n0, s * BK, rb[s % D]);
        }
    __syncthreads();
    read_frags(0, 0, 0);

    auto multiply = [&](int buf) {
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf][i][s], fb[buf][j][s], acc.t[i][j], 0, 0, 0);
    };
    constexpr int MFMAS = 4 * TM * TN;                                   // per fragment set
    constexpr int FRAG_READS = TM + (CFG::B_KMAJOR ? TN : 2 * TN) + (CFG::A_KMAJOR ? 0 : TM);  // LDS read instructions per set (approx.)
    // one slice; MORE: another slice follows (in register slot `slot`); LOAD: the slice D after that
    // one exists and takes its place in the slot
    auto slice = [&](int kt, int slot, auto more_c, auto load_c) {
        constexpr bool MORE = decltype(more_c)::value, LOAD = decltype(load_c)::value;
        const int cur = kt & 1;
#pragma unroll
        for (int q = 0; q < Q; q++) {
            const int buf = q & 1;
            if (q == 0 && MORE) {
                opA::store_lds(stage_a(cur ^ 1), ra[slot]);
                opB::store_lds(stage_b(cur ^ 1), rb[slot]);
                if (LOAD) {
                    opA::load_global(A, m0, (kt + 1 + D) * BK, ra[slot]);
                    opB::load_global(B, n0, (kt + 1 + D) * BK, rb[slot]);
                }
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
            // spread the memory instructions of this block between the matrix instructions
            constexpr int NVS = opA::NV + opB::NV;
            constexpr int USED_FIRST = (MORE ? NVS : 0) + (MORE && LOAD ? NVS : 0) + FRAG_READS;
            constexpr int USED_LAST = MORE ? FRAG_READS : 0;
            if (q == 0 && MORE) {
#pragma unroll
                for (int i = 0; i < NVS; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                }
                if (LOAD) {
#pragma unroll
                    for (int i = 0; i < NVS; i++) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                }
            }
            if (q + 1 < Q || MORE) {
#pragma unroll
                for (int i = 0; i < FRAG_READS; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            }
            // the remaining matrix instructions of the block (the builtin wants a positive constant)
            constexpr int REST_FIRST = MFMAS > USED_FIRST ? MFMAS - USED_FIRST : 1;
            constexpr int REST_LAST = MFMAS > USED_LAST ? MFMAS - USED_LAST : 1;
            constexpr int REST_MID = MFMAS > FRAG_READS ? MFMAS - FRAG_READS : 1;
            if (q == 0) { if (MFMAS > USED_FIRST) __builtin_amdgcn_sched_group_barrier(0x008, REST_FIRST, 0); }
            else if (q + 1 == Q) { if (MFMAS > USED_LAST) __builtin_amdgcn_sched_group_barrier(0x008, REST_LAST, 0); }
            else { if (MFMAS > FRAG_READS) __builtin_amdgcn_sched_group_barrier(0x008, REST_MID, 0); }
        }
    };
    if (D == 1) {
        int kt = 0;
        for (; kt + 2 < KT; kt++) slice(kt, 0, std::true_type(), std::true_type());
        if (kt + 1 < KT) { slice(kt, 0, std::true_type(), std::false_type()); kt++; }
        if (kt < KT) slice(kt, 0, std::false_type(), std::false_type());
    } else {
        // unrolled by D so that every register slot index is a constant
        for (int kt0 = 0; kt0 < KT; kt0 += D) {
#pragma unroll
            for (int d = 0; d < D; d++) {
                const int kt = kt0 + d;
                if (kt >= KT) break;
                if (kt + 1 + D < KT) slice(kt, (d + 1) % D, std::true_type(), std::true_type());
                else if (kt + 1 < KT) slice(kt, (d + 1) % D, std::true_type(), std::false_type());
                else slice(kt, (d + 1) % D, std::false_type(), std::false_type());
            }
        }
    }
    // the next call may overwrite stage 0 while a slow wavefront still multiplies: its fragments are
    // in registers, and the barrier above ordered every LDS read of this call before that
}

// Adds the partial sums of the WGK groups of wavefronts into group 0 (through `lds`, the buffer
// tile_accumulate used: its last barrier ordered every read of it before this).  Returns whether the
// calling wavefront holds the sums, i.e. should run the epilogue.  All threads must call it.
template <class CFG>
__device__ __forceinline__ bool tile_reduce_k(accumulators<CFG> &acc, float *lds) {
    if (CFG::WGK == 1) return true;
    constexpr int WMN = CFG::WGM * CFG::WGN, REGS4 = CFG::TM * CFG::TN * 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wk = wave / WMN, wmn = wave % WMN;
    // slot of (K group g >= 1, wavefront wmn, register quad r): 64 lanes x 16 bytes, conflict-free
    auto slot = [&](int g, int r) -> f32x4 * {
        return reinterpret_cast<f32x4 *>(lds) + (((g - 1) * WMN + wmn) * REGS4 + r) * 64 + lane;
    };
    if (wk > 0) {
#pragma unroll
        for (int i = 0; i < CFG::TM; i++)
#pragma unroll
            for (int j = 0; j < CFG::TN; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const f32x4 v = {acc.t[i][j][4 * r], acc.t[i][j][4 * r + 1], acc.t[i][j][4 * r + 2], acc.t[i][j][4 * r + 3]};
                    *slot(wk, (i * CFG::TN + j) * 4 + r) = v;
                }
    }
    __syncthreads();
    if (wk > 0) return false;
#pragma unroll
    for (int g = 1; g < CFG::WGK; g++)
#pragma unroll
        for (int i = 0; i < CFG::TM; i++)
#pragma unroll
            for (int j = 0; j < CFG::TN; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const f32x4 v = *slot(g, (i * CFG::TN + j) * 4 + r);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc.t[i][j][4 * r + e] += v[e];
                }
    return true;
}

// Hands every element of the tile to the epilogue: epi(row, col, value).  With WGK > 1 only the
// wavefronts for which tile_reduce_k returned true may call it.
template <class CFG, class EPI>
__device__ __forceinline__ void tile_epilogue(const accumulators<CFG> &acc, int M, int N, int m0, int n0, EPI epi) {
    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) % (CFG::WGM * CFG::WGN);
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;
    // accumulator register r of a lane holds row 8*(r/4) + 4*h + r%4, column lane%32 of its tile
#pragma unroll
    for (int i = 0; i < CFG::TM; i++)
#pragma unroll
        for (int j = 0; j < CFG::TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm * CFG::WM + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                const int col = n0 + wn * CFG::WN + j * 32 + l32;
                if (!CFG::EDGE || (row < M && col < N)) epi(row, col, acc.t[i][j][r]);
            }
}

// The epilogue in two passes: value(row, column, sum) returns what the element's store will write (it may read
// memory), store(row, column, v) writes it.  Loads and stores are counted by one in-order counter (vmcnt): a load
// issued behind a store can only be waited for together with that store's acknowledgement, so a tile whose
// elements load and store in turn pays a round trip to memory per element.  Here the values of a group of
// accumulator tiles (64 elements per lane: what the loads of the first pass may keep in registers) are all
// computed before the group's first store is issued: one round trip per group.
template <class CFG, class VALUE, class STORE>
__device__ __forceinline__ void tile_epilogue(accumulators<CFG> &acc, int M, int N, int m0, int n0, VALUE value, STORE store) {
    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) % (CFG::WGM * CFG::WGN);
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;
    constexpr int TILES = CFG::TM * CFG::TN, GROUP = 4;
#pragma unroll
    for (int g0 = 0; g0 < TILES; g0 += GROUP)
#pragma unroll
        for (int pass = 0; pass < 2; pass++)
#pragma unroll
            for (int g = g0; g < g0 + GROUP && g < TILES; g++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int i = g / CFG::TN, j = g % CFG::TN;
                    const int row = m0 + wm * CFG::WM + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                    const int col = n0 + wn * CFG::WN + j * 32 + l32;
                    if (!CFG::EDGE || (row < M && col < N)) {
                        if (pass == 0) acc.t[i][j][r] = value(row, col, acc.t[i][j][r]);
                        else store(row, col, acc.t[i][j][r]);
                    }
                }
}

template <class CFG, class VALUE, class STORE>
__device__ __forceinline__ void tile_mainloop(const float *__restrict__ A, long lda, const float *__restrict__ B,
                                              long ldb, int M, int N, int K, int m0, int n0, bool vec_ok,
                                              float *lds, VALUE value, STORE store) {
    accumulators<CFG> acc;
    acc.clear();
    linear_source<CFG::A_KMAJOR, CFG::EDGE> sa{A, lda, M, K, vec_ok};
    linear_source<CFG::B_KMAJOR, CFG::EDGE> sb{B, ldb, N, K, vec_ok};
    tile_accumulate<CFG>(acc, sa, sb, K, m0, n0, lds);
    if (tile_reduce_k<CFG>(acc, lds)) tile_epilogue<CFG>(acc, M, N, m0, n0, value, store);
}

// C = alpha * sum + beta * C as the two passes of tile_epilogue
struct axpby_value {
    const float *C;
    long ldc;
    float alpha, beta;
    __device__ __forceinline__ float operator()(int row, int col, float v) const {
        return (beta == 0.f) ? alpha * v : alpha * v + beta * C[(long)row * ldc + col];
    }
};
struct axpby_store {
    float *C;
    long ldc;
    __device__ __forceinline__ void operator()(int row, int col, float v) const { C[(long)row * ldc + col] = v; }
};

template <class CFG>
__global__ void __launch_bounds__(CFG::NT) sgemm_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                         float *__restrict__ C, int M, int N, int K, long lda, long ldb,
                                                         long ldc, float alpha, float beta, int vec_ok) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    int tm, tn;
    tile_of_block((M + CFG::BM - 1) / CFG::BM, (N + CFG::BN - 1) / CFG::BN, tm, tn);
    tile_mainloop<CFG>(A, lda, B, ldb, M, N, K, tm * CFG::BM, tn * CFG::BN, vec_ok != 0, lds, axpby_value{C, ldc, alpha, beta},
                       axpby_store{C, ldc});
}

// Up to eight problems of one shape in one launch: blockIdx.z picks the operands.
constexpr int BATCH_MAX = 8;
struct sgemm_batch {
    const float *A[BATCH_MAX];
    const float *B[BATCH_MAX];
    float *C[BATCH_MAX];
};

template <class CFG>
__global__ void __launch_bounds__(CFG::NT) sgemm_batched_kernel(const sgemm_batch batch, int M, int N, int K, long lda, long ldb,
                                                                 long ldc, float alpha, float beta, int vec_ok) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    int tm, tn;
    tile_of_block((M + CFG::BM - 1) / CFG::BM, (N + CFG::BN - 1) / CFG::BN, tm, tn);
    const float *A = batch.A[blockIdx.z], *B = batch.B[blockIdx.z];
    float *C = batch.C[blockIdx.z];
    tile_mainloop<CFG>(A, lda, B, ldb, M, N, K, tm * CFG::BM, tn * CFG::BN, vec_ok != 0, lds, axpby_value{C, ldc, alpha, beta},
                       axpby_store{C, ldc});
}

}  // namespace tgemm
#endif
