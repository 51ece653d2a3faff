// fp32 contraction on the matrix cores whose B operand is a *sliding window* over a tensor -- the
// implicit GEMM of a convolution:
//     C[m, p] = sum over (c, t) of  A[m, c * TAPS + t] * X[ f(p) + c * chan_stride + tap_offset(t) ]
// with p a flattened output position, c a channel and t a tap of the window.  The gathered operand is
// never formed: for a block of CB channels a workgroup copies, per channel, the one contiguous piece
// of X that its BN positions and all taps touch ([f(first p), f(last p) + largest tap offset], WIN
// floats at most) into LDS with coalesced 16-byte loads, and every MFMA operand is then a single LDS
// read at   (lane's position offset) + (compile-time constant of the channel and tap).
//
// Layout in LDS, per stage:  A block as [channel][tap][BM] (lanes read consecutive m), X block as
// [channel][WIN]; both channel strides are = 32 mod 64 floats, so that the two halves of a wavefront
// -- which hold neighbouring channels of the same tap, v_mfma_f32_32x32x2_f32 takes two k per
// instruction -- read from disjoint banks.  Two stages: while the matrix cores work
// on one block of channels, the next one travels global -> registers -> other stage; one barrier
// per block.  The loops over taps and channel pairs are fully unrolled, so tap offsets and channel
// strides end up in the instructions' immediate offsets and the inner loop has no address arithmetic.
//
// Requirements (checked by the emitter): whole tiles (M % BM == 0, N % BN == 0, channels % CB == 0,
// CB even), a tile's positions within one image (so that its window is one short piece of memory),
// channel stride and A's leading dimension multiples of 4, operands 16-byte aligned.
#ifndef TIRAMISU_AMD_GEMM_MFMA_WINDOW_HIP_H
#define TIRAMISU_AMD_GEMM_MFMA_WINDOW_HIP_H
#include "gemm_mfma.hip.h"

namespace tgemm {

// TAP_OFFSETS: a type with  static constexpr int at(int tap)  (offset of a tap within the window).
// POS: a functor  long operator()(int p)  giving f(p), the offset of position p's window origin in X.
// VALUE, STORE: the two passes of tile_epilogue over a finished tile.
//
// Work distribution.  The launch has as many workgroups as the chip holds at a time (one or two per compute
// unit, by their LDS footprint) and they take work items from a queue: first the whole tiles -- all tiles but
// R = T mod G, G = gridDim.x --, then the R remaining tiles cut into SPLITS pieces each along the channel blocks
// (1568 tiles, 512 workgroups: 1536 whole tiles, then 32 tiles as 256 pieces), so that the end of the launch is
// filled with short items.  Items come from atomic counters, one item ahead, because the first block of the next
// item is already travelling while the current item's last block is multiplied.  Two workgroups of a compute unit
// share its matrix pipeline unevenly; with a fixed list per workgroup the slower one would finish its list alone,
// at a workgroup's solo rate.  The whole tiles are dealt to the XCDs in contiguous ranges with a counter each
// (workgroup w runs on XCD w mod 8): the windows of neighbouring tiles overlap -- 544 floats per channel for 256
// positions here -- and are fetched once per L2 when neighbours run on the same XCD at about the same time.  A
// workgroup whose XCD has no whole tile left takes pieces, from one counter for all.
// The pieces of a tile meet in `scratch`: partial tiles, one counter per remaining tile, then the piece queue, a
// counter of finished workgroups and the XCDs' queues (all counters zero between launches; the last workgroup to
// finish zeroes the queues).  The workgroup whose piece arrives last adds the pieces in piece order and runs the
// epilogue, so the result does not depend on the order of arrival.
template <class CFG, int CB, int TAPS, int WIN, int AHEAD, int SPLITS, bool BY_XCD, class TAP_OFFSETS, class POS, class VALUE, class STORE>
__device__ __forceinline__ void contraction_window(const float *__restrict__ A, long lda, const float *__restrict__ X, long x_elements,
                                                   const POS &pos, long chan_stride, int channels, int M, int N,
                                                   float *__restrict__ scratch, float *lds, VALUE value, STORE store) {
    constexpr int BM = CFG::BM, BN = CFG::BN, NT = CFG::NT, TM = CFG::TM, TN = CFG::TN;
    constexpr int KL = CB * TAPS;                         // k per block of channels
    constexpr int A_CHANNEL = TAPS * BM + 32;             // floats per channel of the A block: = 32 mod 64, see above
    constexpr int A_FLOATS = CB * A_CHANNEL, X_FLOATS = CB * WIN, STAGE = A_FLOATS + X_FLOATS;
    constexpr int A_UNITS = BM * KL / 4, X_UNITS = CB * WIN / 4;          // 16-byte pieces per block
    constexpr int NVA = (A_UNITS + NT - 1) / NT, NVX = (X_UNITS + NT - 1) / NT;
    constexpr int STEPS = TAPS * CB / 2;
    static_assert(CB % 2 == 0 && KL % 4 == 0 && WIN % 4 == 0 && WIN % 64 == 32 && (TAPS * BM) % 64 == 0, "block shape");
    static_assert(CFG::WGK == 1, "no K groups in the windowed kernel");
    __shared__ unsigned ticket;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / CFG::WGN, wn = wave % CFG::WGN;
    const int l32 = lane & 31, h = lane >> 5;

    // ---- work items: whole tiles [0, whole), then pieces of the remaining tiles
    const int tiles_m = M / BM, tiles = tiles_m * (N / BN), G = gridDim.x, w = blockIdx.x;
    const int blocks = channels / CB;
    constexpr int splits = SPLITS;
    constexpr bool split = splits > 1;
    const int rest = split ? tiles % G : 0, whole = tiles - rest, items = whole + rest * splits;
    auto is_piece = [&](int q) { return q >= whole; };
    auto item_tile = [&](int q) { return is_piece(q) ? whole + (q - whole) / splits : q; };
    auto item_first = [&](int q) { return is_piece(q) ? (int)((long)((q - whole) % splits) * blocks / splits) : 0; };
    auto item_end = [&](int q) { return is_piece(q) ? (int)((long)((q - whole) % splits + 1) * blocks / splits) : blocks; };

    // ---- one block of channels.  The block in `stage` is multiplied: STEPS steps of TM * TN matrix instructions, each on
    // one tap and one pair of channels (the two halves of a wavefront hold the two channels), the operands of step s + 1
    // requested from LDS before the matrix instructions of step s are issued.  Meanwhile block `next_b` of the tile
    // aimed at (m0_load / f0_load) travels into the other stage: its 16-byte loads are issued during the first steps,
    // their LDS writes during the last ones.  Everything is one basic block -- no predicated loads: the threads past
    // the last 16-byte unit repeat the first ones -- and the scheduling groups deal loads, LDS reads and LDS writes
    // out between the matrix instructions, in whose shadow they cost nothing: with one wavefront per SIMD, whatever is
    // issued while the matrix pipeline is idle is lost time.
    int m0_load = 0;
    long f0_load = 0;
    auto aim_loads_at = [&](int tile) {
        m0_load = (tile % tiles_m) * BM;
        f0_load = pos((tile / tiles_m) * BN) & ~3L;       // window origin, aligned down to 16 bytes
    };
    constexpr int NU = NVA + NVX;                             // 16-byte units per thread and block
    constexpr int PER_STEP = (NU + (STEPS / 2 > 0 ? STEPS / 2 : 1) - 1) / (STEPS / 2 > 0 ? STEPS / 2 : 1);
    constexpr int MOVE_STEPS = (NU + PER_STEP - 1) / PER_STEP, FIRST_WRITE_STEP = STEPS - MOVE_STEPS;
    f32x4 ru[NU];
    auto load_unit = [&](int v, int b) {
        if (v < NVA) {
            const int u = (t + NT * v) % A_UNITS, m = u % BM, k4 = u / BM;
            ru[v] = *reinterpret_cast<const f32x4 *>(A + (long)(m0_load + m) * lda + (long)b * KL + 4 * k4);
        } else {
            const int u = (t + NT * (v - NVA)) % X_UNITS, c = u / (WIN / 4), w4 = u % (WIN / 4);
            long at = f0_load + ((long)b * CB + c) * chan_stride + 4 * w4;
            // the tail of the last window may lie beyond the tensor: those floats are never used
            at = at + 3 < x_elements ? at : 0;
            ru[v] = *reinterpret_cast<const f32x4 *>(X + at);
        }
    };
    auto write_unit = [&](int v, int stage) {
        float *la = lds + stage * STAGE, *lx = la + A_FLOATS;
        if (v < NVA) {
            const int u = (t + NT * v) % A_UNITS, m = u % BM, k4 = u / BM;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int kl = 4 * k4 + e;                                // = channel * TAPS + tap
                la[(kl / TAPS) * A_CHANNEL + (kl % TAPS) * BM + m] = ru[v][e];
            }
        } else {
            const int u = (t + NT * (v - NVA)) % X_UNITS;
            *reinterpret_cast<f32x4 *>(lx + 4 * u) = ru[v];
        }
    };
    accumulators<CFG> acc;
    int fp[TN];                                               // lane's position offsets in the current tile's window
    const int arow = wm * CFG::WM + l32 + h * A_CHANNEL;
    constexpr int RING = AHEAD + 1;                           // operands are requested from LDS AHEAD steps before their use
    float fa[RING][TM], fb[RING][TN];
    auto read_step = [&](int stage, int st, int buf) {
        const float *la = lds + stage * STAGE + arow, *lx = lds + stage * STAGE + A_FLOATS;
        const int tap = st / (CB / 2), c = 2 * (st % (CB / 2));
#pragma unroll
        for (int i = 0; i < TM; i++) fa[buf][i] = la[c * A_CHANNEL + tap * BM + i * 32];
#pragma unroll
        for (int j = 0; j < TN; j++) fb[buf][j] = lx[fp[j] + c * WIN + TAP_OFFSETS::at(tap)];
    };
    auto block = [&](int stage, int next_b) {
#pragma unroll
        for (int st = 0; st < AHEAD && st < STEPS; st++) read_step(stage, st, st % RING);
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            const int buf = st % RING;
#pragma unroll
            for (int v = st * PER_STEP; v < (st + 1) * PER_STEP && v < NU; v++) load_unit(v, next_b);
            if (st + AHEAD < STEPS) read_step(stage, st + AHEAD, (st + AHEAD) % RING);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf][i], fb[buf][j], acc.t[i][j], 0, 0, 0);
            if (st >= FIRST_WRITE_STEP)
#pragma unroll
                for (int v = (st - FIRST_WRITE_STEP) * PER_STEP; v < (st - FIRST_WRITE_STEP + 1) * PER_STEP && v < NU; v++) write_unit(v, stage ^ 1);
            // the order of this step's instructions: its loads, LDS reads and matrix instructions in turn, the rest of
            // the matrix instructions but one, its LDS writes, the last matrix instruction
#pragma unroll
            for (int v = st * PER_STEP; v < (st + 1) * PER_STEP && v < NU; v++) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            const int between_reads = st + AHEAD < STEPS ? (TM + TN < TM * TN - 1 ? TM + TN : TM * TN - 1) : 0;
            if (st + AHEAD < STEPS)
#pragma unroll
                for (int r = 0; r < TM + TN; r++) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (r < between_reads) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
#pragma unroll
            for (int q = between_reads; q < TM * TN - 1; q++) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (st >= FIRST_WRITE_STEP)
#pragma unroll
                for (int v = (st - FIRST_WRITE_STEP) * PER_STEP; v < (st - FIRST_WRITE_STEP + 1) * PER_STEP && v < NU; v++)
#pragma unroll
                    for (int e = 0; e < (v < NVA ? 4 : 1); e++) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __syncthreads();
    };
    auto aim_tile_at = [&](int tile, int &m0, int &n0) {
        m0 = (tile % tiles_m) * BM;
        n0 = (tile / tiles_m) * BN;
        const long f0 = pos(n0) & ~3L;
#pragma unroll
        for (int j = 0; j < TN; j++) fp[j] = (int)(pos(n0 + wn * CFG::WN + j * 32 + l32) - f0) + h * WIN;
    };

    // ---- a piece of a remaining tile: park it in scratch; the last piece to arrive adds all of them
    constexpr int QUADS = TM * TN * 4;
    f32x4 *pieces = reinterpret_cast<f32x4 *>(scratch);
    unsigned *counters = reinterpret_cast<unsigned *>(scratch + (long)rest * splits * BM * BN);
    unsigned *piece_queue = counters + rest, *finished = piece_queue + 1, *xcd_queue = finished + 1;
    auto finish_piece = [&](int q, int m0, int n0) {
        const int rt = (q - whole) / splits, z = (q - whole) % splits;
        f32x4 *mine = pieces + ((long)rt * splits + z) * QUADS * NT;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    store_handed_over(mine + ((i * TN + j) * 4 + r) * NT + t, f32x4{acc.t[i][j][4 * r], acc.t[i][j][4 * r + 1], acc.t[i][j][4 * r + 2], acc.t[i][j][4 * r + 3]});
        handed_over_stores_done();         // the piece is in memory before the ticket is taken
        __syncthreads();
        if (t == 0) ticket = atomicAdd(&counters[rt], 1u);
        __syncthreads();
        if (ticket != (unsigned)(splits - 1)) return;
        handed_over_loads_begin();
        // a rolled loop over pairs of quads (no accumulator registers involved: the element's place follows from the
        // quad's index, as in tile_epilogue); all pieces of a pair are requested before the first is added, so that a
        // pair costs one round trip to memory, and they are added in piece order
        const f32x4 *all = pieces + (long)rt * splits * QUADS * NT;
#pragma unroll 1
        for (int q0 = 0; q0 < QUADS; q0 += 2) {
            f32x4 part[2][SPLITS];
#pragma unroll
            for (int c = 0; c < SPLITS; c++)
#pragma unroll
                for (int d = 0; d < 2; d++)
                    part[d][c] = load_handed_over(all + ((long)c * QUADS + q0 + d) * NT + t);
#pragma unroll
            for (int d = 0; d < 2; d++) {
                f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < SPLITS; c++) sum += part[d][c];
                const int q = q0 + d, i = q / (4 * TN), j = (q / 4) % TN, r = q % 4;
                const int col = n0 + wn * CFG::WN + j * 32 + l32;
#pragma unroll
                for (int e = 0; e < 4; e++) sum[e] = value(m0 + wm * CFG::WM + i * 32 + 8 * r + 4 * h + e, col, sum[e]);
#pragma unroll
                for (int e = 0; e < 4; e++) store(m0 + wm * CFG::WM + i * 32 + 8 * r + 4 * h + e, col, sum[e]);
            }
        }
        if (t == 0) counters[rt] = 0;      // zero again for the next launch
    };

    __shared__ int next_item;
    // this workgroup's group (its XCD), its place there, the group's range of whole tiles
    const int groups = BY_XCD && G % ttarget::XCDS == 0 ? ttarget::XCDS : 1, x = w % groups, in_group = G / groups;
    const int lo = (int)((long)x * whole / groups), hi = (int)((long)(x + 1) * whole / groups);
    auto take_item = [&]() {
        const int i = in_group + (int)atomicAdd(xcd_queue + x, 1u);
        return lo + i < hi ? lo + i : whole + (int)atomicAdd(piece_queue, 1u);
    };
    int cur = lo + w / groups;                     // G <= whole: every workgroup has a first item
    int m0, n0;
    aim_loads_at(item_tile(cur));
    aim_tile_at(item_tile(cur), m0, n0);
    acc.clear();
#pragma unroll
    for (int v = 0; v < NU; v++) load_unit(v, item_first(cur));
#pragma unroll
    for (int v = 0; v < NU; v++) write_unit(v, 0);
    __syncthreads();
    int stage = 0;
    while (cur < items) {
        // the item after this one (a barrier lies between this write and the previous item's read: block() has one)
        if (t == 0) next_item = take_item();
        __syncthreads();
        const int next = next_item;
        // all blocks but the last: nothing but the block pipeline in this loop
        const int b_end = item_end(cur);
        for (int b = item_first(cur); b + 1 < b_end; b++) {
            block(stage, b + 1);
            stage ^= 1;
        }
        // the last block, with the first block of the next item travelling (of this item again when there is none:
        // loaded and never used)
        const int then = next < items ? next : cur;
        aim_loads_at(item_tile(then));
        block(stage, item_first(then));
        stage ^= 1;
        if (!is_piece(cur)) tile_epilogue<CFG>(acc, M, N, m0, n0, value, store);
        else finish_piece(cur, m0, n0);
        acc.clear();
        aim_tile_at(item_tile(then), m0, n0);
        cur = next;
    }
    // the last workgroup to run out of items leaves the queue ready for the next launch
    if (t == 0 && atomicAdd(finished, 1u) == (unsigned)(G - 1)) {
        *piece_queue = 0;
        *finished = 0;
        for (int g = 0; g < groups; g++) xcd_queue[g] = 0;
    }
}

}  // namespace tgemm
#endif
