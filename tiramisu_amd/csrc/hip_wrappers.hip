// Runtime layer between generated Tiramisu host code and HIP: the C ABI declared in
// include/tiramisu_hip_wrappers.h.  Replaces src/tiramisu_cuda_wrappers.cpp of the reference
// (same failure model: print and exit(1)), adds code-object loading and kernel launch so that
// generated host code needs no HIP headers, and implements the GEMM library call with this
// build's own MFMA kernel instead of a vendor BLAS.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../include/tiramisu_hip_wrappers.h"
#include "kernels/gemm_mfma.hip.h"
#include "kernels/gemm_mfma_f64.hip.h"
#include "kernels/target_gfx950.h"

namespace {

inline void check(hipError_t e, const char *fn) {
    if (e != hipSuccess) {
        fprintf(stderr, "Error at %s: %s\n", fn, hipGetErrorString(e));
        exit(1);
    }
}

thread_local hipStream_t current_stream = hipStreamPerThread;

// ---- per-launch timing records
struct launch_record {
    std::string name;
    hipEvent_t start, stop;
    float ms;
};
std::atomic<bool> profiling{false};
std::vector<launch_record> records;     // guarded by records_mutex: launches may come from pool threads
std::mutex records_mutex;
std::mutex names_mutex;
std::map<void *, std::string> function_names;

struct scoped_record {
    bool on;
    scoped_record(const std::string &name) : on(profiling) {
        if (!on) return;
        launch_record r;
        r.name = name;
        r.ms = 0.f;
        check(hipEventCreate(&r.start), "tiramisu_hip_profile");
        check(hipEventCreate(&r.stop), "tiramisu_hip_profile");
        check(hipEventRecord(r.start, current_stream), "tiramisu_hip_profile");
        stop = r.stop;
        std::lock_guard<std::mutex> g(records_mutex);
        records.push_back(r);
    }
    ~scoped_record() {
        if (on) check(hipEventRecord(stop, current_stream), "tiramisu_hip_profile");
    }
    hipEvent_t stop = nullptr;
};

// ---- pool for host loops tagged parallel.  Threads are created on first use and live until
// the process ends (the state is never destroyed, so nothing is torn down under a waiting thread).
struct parallel_pool {
    // as many as there are hardware queues per process by default; TIRAMISU_HIP_POOL_THREADS overrides (1..16)
    const int WORKERS = [] {
        const char *e = std::getenv("TIRAMISU_HIP_POOL_THREADS");
        const int n = e ? std::atoi(e) : 4;
        return n < 1 ? 1 : n > 16 ? 16 : n;
    }();
    std::mutex m;
    std::condition_variable wake, done;
    std::vector<std::thread> threads;
    // the job being run (one at a time: jobs_mutex serialises callers)
    std::mutex jobs_mutex;
    void (*body)(int32_t, void *) = nullptr;
    void *closure = nullptr;
    int32_t next = 0, last = -1;
    long generation = 0;
    int active = 0;
    int device = 0;        // the device that was current when the pool was first used

    void worker() {
        check(hipSetDevice(device), "tiramisu_hip_parallel_for");
        hipStream_t s;
        check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "tiramisu_hip_parallel_for");
        current_stream = s;
        long seen = 0;
        std::unique_lock<std::mutex> lk(m);
        for (;;) {
            wake.wait(lk, [&] { return generation != seen; });
            seen = generation;
            while (next <= last) {
                const int32_t i = next++;
                lk.unlock();
                body(i, closure);
                lk.lock();
            }
            lk.unlock();
            check(hipStreamSynchronize(s), "tiramisu_hip_parallel_for");
            lk.lock();
            if (--active == 0) done.notify_all();
        }
    }

    void run(int32_t first, int32_t last_, void (*b)(int32_t, void *), void *c) {
        std::lock_guard<std::mutex> one(jobs_mutex);
        std::unique_lock<std::mutex> lk(m);
        if (threads.empty()) check(hipGetDevice(&device), "tiramisu_hip_parallel_for");
        while ((int)threads.size() < WORKERS) {
            threads.emplace_back([this] { worker(); });
            threads.back().detach();
        }
        body = b;
        closure = c;
        next = first;
        last = last_;
        active = WORKERS;
        generation++;
        wake.notify_all();
        done.wait(lk, [&] { return active == 0; });
    }
};
thread_local bool in_parallel_iteration = false;

// ---- pooled device memory (see tiramisu_hip_malloc)
std::mutex pool_mutex;
std::map<uint64_t, std::vector<void *>> pool_free;   // idle blocks by size
std::map<void *, uint64_t> pool_live;                  // blocks handed out
uint64_t pool_idle_bytes = 0;
uint64_t pool_limit() {
    static const uint64_t limit = [] {
        const char *e = std::getenv("TIRAMISU_HIP_POOL_BYTES");
        return e ? (uint64_t)std::strtoull(e, nullptr, 10) : (uint64_t)16 << 30;
    }();
    return limit;
}

// One thread per element of C; any strides, any sizes.  Used for double precision and for
// shapes the MFMA path does not take.
template <typename T>
__global__ void gemm_generic_kernel(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, int M, int N,
                                    int K, long a_rs, long a_cs, long b_rs, long b_cs, long ldc, T alpha, T beta) {
    const int col = blockIdx.x * blockDim.x + threadIdx.x;
    const int row = blockIdx.y * blockDim.y + threadIdx.y;
    if (row >= M || col >= N) return;
    T acc = 0;
    for (int k = 0; k < K; k++) acc += A[row * a_rs + k * a_cs] * B[k * b_rs + col * b_cs];
    T *p = C + (long)row * ldc + col;
    *p = (beta == (T)0) ? alpha * acc : alpha * acc + beta * *p;
}

// Problems of one shape gathered by a batch scope (tiramisu_hip_batch_begin / _end) that the next MFMA launch of
// this thread covers in one go, one problem per blockIdx.z.
thread_local const tgemm::sgemm_batch *active_batch = nullptr;
thread_local int active_batch_count = 0;

template <class CFG>
void launch_mfma(const float *A, const float *B, float *C, int M, int N, int K, long lda, long ldb, long ldc,
                 float alpha, float beta, bool vec_ok) {
    const int tiles = ((M + CFG::BM - 1) / CFG::BM) * ((N + CFG::BN - 1) / CFG::BN);
    if (active_batch) {
        hipLaunchKernelGGL((tgemm::sgemm_batched_kernel<CFG>), dim3(tiles, 1, active_batch_count), dim3(CFG::NT), CFG::LDS_BYTES, current_stream,
                           *active_batch, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok ? 1 : 0);
        check(hipGetLastError(), "tiramisu_hip_sgemm");
        return;
    }
    hipLaunchKernelGGL((tgemm::sgemm_kernel<CFG>), dim3(tiles), dim3(CFG::NT), CFG::LDS_BYTES, current_stream, A, B, C,
                       M, N, K, lda, ldb, ldc, alpha, beta, vec_ok ? 1 : 0);
    check(hipGetLastError(), "tiramisu_hip_sgemm");
}

// The square C tile whose launch is modelled fastest on this machine.
int tile_for(int M, int N) { return ttarget::square_tile_for(M, N); }

template <bool AK, bool BK_, bool EDGE>
void dispatch_tile(const float *A, const float *B, float *C, int M, int N, int K, long lda, long ldb, long ldc,
                   float alpha, float beta, bool vec_ok) {
    const int bm = tile_for(M, N);
    if constexpr (!EDGE) {
        if (bm == 256)
            return launch_mfma<tgemm::config<256, 256, 16, 2, 2, AK, BK_, false, 0>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
        if (bm == 192)
            return launch_mfma<tgemm::config<192, 192, 16, 2, 2, AK, BK_, false>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
    }
    if (bm == 128)
        launch_mfma<tgemm::config<128, 128, 16, 2, 2, AK, BK_, EDGE>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
    else
        launch_mfma<tgemm::config<64, 64, 32, 2, 2, AK, BK_, EDGE>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
}

// Few C tiles but a long reduction (a batch of 64 rows against wide weights, as in recurrent
// cells): 64x32 tiles, 8 groups of wavefronts share the K range of each tile and reduce through
// LDS, and up to four K-slices are requested ahead (the launch is latency-bound).
bool skinny(int M, int N, int K, bool vec_ok, bool transposeA) {
    return !transposeA && vec_ok && M == 64 && (N + 63) / 64 <= ttarget::COMPUTE_UNITS / 4 && N % 32 == 0 && K % 128 == 0 && K >= 256;
}

template <bool BK_>
void dispatch_skinny(const float *A, const float *B, float *C, int M, int N, int K, long lda, long ldb, long ldc,
                     float alpha, float beta) {
    // K = 512 (the recurrent product of a 512-unit cell): four groups of wavefronts, 64-k slices, one slice ahead
    // (9.2 us per call against 10.9 us for the eight-group form below)
    if (K == 512) return launch_mfma<tgemm::config<64, 32, 64, 2, 1, true, BK_, false, 0, 4, 1>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, true);
    switch (std::min(4, K / 128 - 1)) {
    case 1: return launch_mfma<tgemm::config<64, 32, 128, 2, 1, true, BK_, false, 0, 8, 1>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, true);
    case 2: return launch_mfma<tgemm::config<64, 32, 128, 2, 1, true, BK_, false, 0, 8, 2>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, true);
    case 3: return launch_mfma<tgemm::config<64, 32, 128, 2, 1, true, BK_, false, 0, 8, 3>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, true);
    default: return launch_mfma<tgemm::config<64, 32, 128, 2, 1, true, BK_, false, 0, 8, 4>>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, true);
    }
}

// ---- deep reductions: the K range split over workgroups.
// A problem with few C tiles and a long K (256 x 256 x 65536: sixteen 64x64 tiles) leaves most of the
// chip idle when one workgroup walks the whole K range of a tile.  Here gridDim.y workgroups take a
// chunk of K each for the same tile, write their partial tile to a scratch buffer, and the last one to
// finish (a counter per tile) adds the partial tiles in chunk order -- so the result does not depend on
// which workgroup came last -- and applies alpha / beta.  No workgroup waits for another.
// Scratch layout: floats [tile][chunk][register quad][thread][4], then one 32-bit counter per tile
// (zero before the launch; the last workgroup leaves it zero again).
constexpr int SPLITK_TILE = 64, SPLITK_THREADS = 256, SPLITK_MAX_TILES = 128;
constexpr uint64_t SPLITK_COUNTER_BYTES = SPLITK_MAX_TILES * sizeof(unsigned);

template <class CFG>
__global__ void __launch_bounds__(CFG::NT) sgemm_splitk_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                                float *__restrict__ C, int M, int N, int K, long lda, long ldb,
                                                                long ldc, float alpha, float beta, int vec_ok, int chunk,
                                                                float *__restrict__ partial, unsigned *__restrict__ counters) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ unsigned ticket;
    static_assert(CFG::WGK == 1 && CFG::TM == 1 && CFG::TN == 1, "one accumulator tile per wavefront");
    int tm, tn;
    const int tiles_n = (N + CFG::BN - 1) / CFG::BN;
    tm = blockIdx.x / tiles_n;
    tn = blockIdx.x % tiles_n;
    const int z = blockIdx.y, Z = gridDim.y;
    const int k0 = z * chunk, kc = min(chunk, K - k0);
    tgemm::accumulators<CFG> acc;
    acc.clear();
    tgemm::linear_source<CFG::A_KMAJOR, CFG::EDGE> sa{A + (CFG::A_KMAJOR ? (long)k0 : (long)k0 * lda), lda, M, kc, vec_ok != 0};
    tgemm::linear_source<CFG::B_KMAJOR, CFG::EDGE> sb{B + (CFG::B_KMAJOR ? (long)k0 : (long)k0 * ldb), ldb, N, kc, vec_ok != 0};
    tgemm::tile_accumulate<CFG>(acc, sa, sb, kc, tm * CFG::BM, tn * CFG::BN, lds);
    tgemm::f32x4 *mine = reinterpret_cast<tgemm::f32x4 *>(partial) + ((long)blockIdx.x * Z + z) * 4 * CFG::NT;
#pragma unroll
    for (int r = 0; r < 4; r++)
        tgemm::store_handed_over(mine + r * CFG::NT + threadIdx.x, tgemm::f32x4{acc.t[0][0][4 * r], acc.t[0][0][4 * r + 1], acc.t[0][0][4 * r + 2], acc.t[0][0][4 * r + 3]});
    tgemm::handed_over_stores_done();      // the partial tile is in memory before the ticket is taken
    __syncthreads();
    if (threadIdx.x == 0) ticket = atomicAdd(&counters[blockIdx.x], 1u);
    __syncthreads();
    if (ticket != (unsigned)(Z - 1)) return;
    tgemm::handed_over_loads_begin();
    const tgemm::f32x4 *all = reinterpret_cast<const tgemm::f32x4 *>(partial) + (long)blockIdx.x * Z * 4 * CFG::NT;
    // four chunks' partial tiles are requested before the first is added (one round trip to memory per four
    // chunks); they are added in chunk order, whichever workgroup arrives last
    tgemm::f32x4 sum[4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int c0 = 0; c0 < Z; c0 += 4) {
        tgemm::f32x4 part[4][4];
#pragma unroll
        for (int cc = 0; cc < 4; cc++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (c0 + cc < Z) part[cc][r] = tgemm::load_handed_over(all + ((long)(c0 + cc) * 4 + r) * CFG::NT + threadIdx.x);
#pragma unroll
        for (int cc = 0; cc < 4; cc++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (c0 + cc < Z) sum[r] += part[cc][r];
    }
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc.t[0][0][4 * r + e] = sum[r][e];
    tgemm::tile_epilogue<CFG>(acc, M, N, tm * CFG::BM, tn * CFG::BN, tgemm::axpby_value{C, ldc, alpha, beta}, tgemm::axpby_store{C, ldc});
    if (threadIdx.x == 0) counters[blockIdx.x] = 0;     // ready for the next launch
}

__global__ void clear_counters_kernel(unsigned *counters, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counters[i] = 0;
}

// How a problem is split: chunks of K (a multiple of the 32-k slice) and the scratch it needs; chunks == 1: not split.
struct splitk_plan {
    int tiles = 0, chunks = 1, chunk = 0;
    uint64_t scratch_bytes = 0;    // partial tiles + counters
};

splitk_plan plan_splitk(int M, int N, int K, uint64_t max_bytes) {
    splitk_plan p;
    p.tiles = ((M + SPLITK_TILE - 1) / SPLITK_TILE) * ((N + SPLITK_TILE - 1) / SPLITK_TILE);
    if (p.tiles > SPLITK_MAX_TILES || K < 2048) return p;
    // enough workgroups for every compute unit, at least 512 of K each
    int chunks = std::min((ttarget::COMPUTE_UNITS + p.tiles - 1) / p.tiles, K / 512);
    const uint64_t per_chunk = (uint64_t)p.tiles * SPLITK_TILE * SPLITK_TILE * sizeof(float);
    while (chunks > 1 && per_chunk * chunks + SPLITK_COUNTER_BYTES > max_bytes) chunks--;
    if (chunks < 2) return p;
    p.chunk = ((K + chunks - 1) / chunks + 31) / 32 * 32;
    p.chunks = (K + p.chunk - 1) / p.chunk;
    p.scratch_bytes = per_chunk * p.chunks + SPLITK_COUNTER_BYTES;
    return p;
}

template <bool AK, bool BK_, bool EDGE>
void launch_splitk(const splitk_plan &p, const float *A, const float *B, float *C, int M, int N, int K, long lda, long ldb, long ldc,
                   float alpha, float beta, bool vec_ok, void *scratch) {
    typedef tgemm::config<SPLITK_TILE, SPLITK_TILE, 32, 2, 2, AK, BK_, EDGE> CFG;
    static_assert(CFG::NT == SPLITK_THREADS, "scratch layout assumes 256 threads");
    unsigned *counters = reinterpret_cast<unsigned *>(scratch);
    float *partial = reinterpret_cast<float *>(reinterpret_cast<char *>(scratch) + SPLITK_COUNTER_BYTES);
    hipLaunchKernelGGL(clear_counters_kernel, dim3(1), dim3(SPLITK_MAX_TILES), 0, current_stream, counters, p.tiles);
    hipLaunchKernelGGL((sgemm_splitk_kernel<CFG>), dim3(p.tiles, p.chunks), dim3(CFG::NT), CFG::LDS_BYTES, current_stream, A, B, C,
                       M, N, K, lda, ldb, ldc, alpha, beta, vec_ok ? 1 : 0, p.chunk, partial, counters);
    check(hipGetLastError(), "tiramisu_hip_sgemm");
}

void dispatch_splitk(const splitk_plan &p, bool tA, bool tB, bool edge, const float *A, const float *B, float *C, int M, int N, int K,
                     long lda, long ldb, long ldc, float alpha, float beta, bool vec_ok, void *scratch) {
#define SPLITK_CASE(AK, BKM)                                                                                              \
    if (edge) launch_splitk<AK, BKM, true>(p, A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok, scratch);              \
    else launch_splitk<AK, BKM, false>(p, A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok, scratch)
    if (!tA && !tB) { SPLITK_CASE(true, false); }
    else if (!tA && tB) { SPLITK_CASE(true, true); }
    else if (tA && !tB) { SPLITK_CASE(false, false); }
    else { SPLITK_CASE(false, true); }
#undef SPLITK_CASE
}

// Scratch of the allocating entry point: one block per host thread and stream (a call works on the thread's
// current stream, and two calls of one thread on two streams may run at the same time: they must not share partial
// tiles and counters), grown on demand, kept until the process ends.
struct splitk_block { void *ptr = nullptr; uint64_t bytes = 0; };
// (the per-thread default stream is one handle that names a different stream in every thread, hence the thread in the key)
typedef std::pair<std::thread::id, hipStream_t> thread_and_stream;
thread_and_stream here() { return {std::this_thread::get_id(), current_stream}; }
std::mutex kept_mutex;                                                    // guards the two maps below
std::map<thread_and_stream, splitk_block> splitk_workspaces;
// Scratch that generated functions keep between their calls (tiramisu_hip_kept_scratch): by requesting site, thread and stream.
std::map<std::pair<const void *, thread_and_stream>, splitk_block> kept_scratch;
constexpr uint64_t SPLITK_WORKSPACE_LIMIT = (uint64_t)256 << 20;

// Scratch of the entry point that allocates nothing: lives in the code object, one copy per device.
constexpr uint64_t STATIC_SCRATCH_BYTES = ((uint64_t)4 << 20) + SPLITK_COUNTER_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
std::mutex static_scratch_mutex;
std::map<int, void *> static_scratch_of_device;      // device -> address of its copy of `scratch`

void *static_scratch_here() {
    int device = 0;
    check(hipGetDevice(&device), "tiramisu_hip_sgemm_static_scratch");
    std::lock_guard<std::mutex> g(static_scratch_mutex);
    auto it = static_scratch_of_device.find(device);
    if (it != static_scratch_of_device.end()) return it->second;
    void *ptr = nullptr;
    check(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "tiramisu_hip_sgemm_static_scratch");
    static_scratch_of_device[device] = ptr;
    return ptr;
}

template <bool AK, bool BK_>
void dispatch_edge(bool edge, const float *A, const float *B, float *C, int M, int N, int K, long lda, long ldb,
                   long ldc, float alpha, float beta, bool vec_ok) {
    if (edge) dispatch_tile<AK, BK_, true>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
    else dispatch_tile<AK, BK_, false>(A, B, C, M, N, K, lda, ldb, ldc, alpha, beta, vec_ok);
}

template <class S, bool A_KFAST, bool B_NFAST>
void launch_dgemm_kernel(const double *A, const double *B, double *C, int M, int N, int K, long sam, long sak, long sbk, long sbn, long ldc,
                                double alpha, double beta) {
    auto kernel = tgemm64::dgemm_kernel<S, A_KFAST, B_NFAST>;
    // the large tile's two LDS stages exceed the 64 KiB that a launch gets without asking (once per device)
    static std::atomic<unsigned long long> asked{0};
    if (S::LDS_BYTES > 64 * 1024) {
        int device = 0;
        check(hipGetDevice(&device), "tiramisu_hip_dgemm");
        const unsigned long long bit = 1ull << (device & 63);
        if (!(asked.load() & bit)) {
            check(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES), "tiramisu_hip_dgemm");
            asked.fetch_or(bit);
        }
    }
    const unsigned tiles = (unsigned)(((M + S::BM - 1) / S::BM) * ((N + S::BN - 1) / S::BN));
    hipLaunchKernelGGL(kernel, dim3(tiles), dim3(S::NT), S::LDS_BYTES, current_stream, A, B, C, M, N, K, sam, sak, sbk, sbn, ldc, alpha, beta);
    check(hipGetLastError(), "tiramisu_hip_dgemm");
}

template <class S>
void launch_dgemm(bool transposeA, bool transposeB, const double *A, const double *B, double *C, int M, int N, int K, long sam, long sak,
                         long sbk, long sbn, long ldc, double alpha, double beta) {
    // A's k is the unit stride unless A is transposed; B's n is unless B is transposed
    if (!transposeA && !transposeB) launch_dgemm_kernel<S, true, true>(A, B, C, M, N, K, sam, sak, sbk, sbn, ldc, alpha, beta);
    else if (!transposeA && transposeB) launch_dgemm_kernel<S, true, false>(A, B, C, M, N, K, sam, sak, sbk, sbn, ldc, alpha, beta);
    else if (transposeA && !transposeB) launch_dgemm_kernel<S, false, true>(A, B, C, M, N, K, sam, sak, sbk, sbn, ldc, alpha, beta);
    else launch_dgemm_kernel<S, false, false>(A, B, C, M, N, K, sam, sak, sbk, sbn, ldc, alpha, beta);
}

}  // namespace

extern "C" {

// Device memory is pooled: generated functions allocate their temporaries on entry and free
// them on exit, every call (the reference pays cudaMalloc / cudaFree each time,
// tiramisu_cuda_wrappers.cpp:55-68).  A freed block is kept, by size, for the next request of that
// size; blocks beyond TIRAMISU_HIP_POOL_BYTES (default 16 GiB; 0 turns pooling off) go back to HIP.
void *tiramisu_hip_malloc(uint64_t size) {
    {
        std::lock_guard<std::mutex> g(pool_mutex);
        auto it = pool_free.find(size);
        if (it != pool_free.end() && !it->second.empty()) {
            void *p = it->second.back();
            it->second.pop_back();
            pool_idle_bytes -= size;
            pool_live[p] = size;
            return p;
        }
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, size);
    if (e == hipErrorOutOfMemory) {
        // give the idle blocks back to HIP and try once more
        (void)hipGetLastError();
        {
            std::lock_guard<std::mutex> g(pool_mutex);
            for (auto &kv : pool_free)
                for (void *q : kv.second) check(hipFree(q), __FUNCTION__);
            pool_free.clear();
            pool_idle_bytes = 0;
        }
        e = hipMalloc(&p, size);
    }
    check(e, __FUNCTION__);
    std::lock_guard<std::mutex> g(pool_mutex);
    pool_live[p] = size;
    return p;
}

int tiramisu_hip_free(void *ptr) {
    if (!ptr) return 0;
    uint64_t size = 0;
    bool keep = false;
    {
        std::lock_guard<std::mutex> g(pool_mutex);
        auto it = pool_live.find(ptr);
        if (it != pool_live.end()) {
            size = it->second;
            pool_live.erase(it);
            keep = pool_idle_bytes + size <= pool_limit();
        }
    }
    if (!keep) {
        check(hipFree(ptr), __FUNCTION__);
        return 0;
    }
    // work that still uses the block was issued on the calling thread's stream (or on pool
    // streams that tiramisu_hip_parallel_for has already synchronised)
    check(hipStreamSynchronize(current_stream), __FUNCTION__);
    std::lock_guard<std::mutex> g(pool_mutex);
    pool_free[size].push_back(ptr);
    pool_idle_bytes += size;
    return 0;
}

int tiramisu_hip_memcpy_to_device(void *to, void *from, uint64_t size) {
    check(hipMemcpyAsync(to, from, size, hipMemcpyHostToDevice, current_stream), __FUNCTION__);
    check(hipStreamSynchronize(current_stream), __FUNCTION__);
    return 0;
}

int tiramisu_hip_memcpy_to_host(void *to, void *from, uint64_t size) {
    check(hipMemcpyAsync(to, from, size, hipMemcpyDeviceToHost, current_stream), __FUNCTION__);
    check(hipStreamSynchronize(current_stream), __FUNCTION__);
    return 0;
}

int tiramisu_hip_memcpy_device_to_device(void *to, void *from, uint64_t size) {
    check(hipMemcpyAsync(to, from, size, hipMemcpyDeviceToDevice, current_stream), __FUNCTION__);
    return 0;
}

int tiramisu_hip_memcpy_to_symbol(void *to, void *from, uint64_t size) {
    // `to` is the device address of the symbol (generated code resolves it when it loads
    // its code object), so this is an ordinary host-to-device copy.
    check(hipMemcpyAsync(to, from, size, hipMemcpyHostToDevice, current_stream), __FUNCTION__);
    check(hipStreamSynchronize(current_stream), __FUNCTION__);
    return 0;
}

int32_t tiramisu_hip_stream_synchronize(int32_t) {
    check(hipStreamSynchronize(current_stream), __FUNCTION__);
    return 0;
}

// Shared by the two single-precision entry points.  `static_scratch`: deep reductions take their scratch
// from the code object's static array and nothing is allocated; else from the calling thread's workspace.
// ---- batch scope: between tiramisu_hip_batch_begin and _end the thread's tiramisu_hip_sgemm calls are gathered
// instead of launched; _end launches runs of calls with one shape (sizes, leading dimensions, transposition, alpha,
// beta, alignment) that go to the MFMA kernels as one launch each (up to tgemm::BATCH_MAX problems per launch) and
// everything else one by one, in call order.
struct gathered_sgemm {
    const float *a, *b;
    float *c;
    uint64_t M, N, K;
    float alpha, beta;
    uint64_t ldA, ldB, ldC;
    bool tA, tB, vec_ok, to_mfma;
    bool same_shape(const gathered_sgemm &o) const {
        return M == o.M && N == o.N && K == o.K && alpha == o.alpha && beta == o.beta && ldA == o.ldA && ldB == o.ldB && ldC == o.ldC &&
               tA == o.tA && tB == o.tB && vec_ok == o.vec_ok && to_mfma == o.to_mfma;
    }
};
thread_local bool batch_open = false;
thread_local std::vector<gathered_sgemm> batch_calls;

static int sgemm_impl(const char *fn, bool static_scratch, float *A, float *B, float *C, uint64_t M, uint64_t N, uint64_t K, float alpha,
                      float beta, uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA, uint64_t offsetB, uint64_t offsetC,
                      bool transposeA, bool transposeB) {
    if (ldA == 0) ldA = transposeA ? M : K;
    if (ldB == 0) ldB = transposeB ? K : N;
    if (ldC == 0) ldC = N;
    if (M == 0 || N == 0) return 0;
    const float *a = A + offsetA, *b = B + offsetB;
    float *c = C + offsetC;
    if (M > 0x7fffffffull || N > 0x7fffffffull || K > 0x7fffffffull) {
        fprintf(stderr, "Error at %s: dimension exceeds 2^31-1\n", fn);
        exit(1);
    }
    const int m = (int)M, n = (int)N, k = (int)K;
    const bool vec_ok = (ldA % 4 == 0) && (ldB % 4 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0);
    const bool small = (m < 32 || n < 32 || k < 8);
    if (batch_open && !static_scratch) {
        // inside a batch scope: remember the call; tiramisu_hip_batch_end launches it, together with the calls of
        // the same shape that follow it
        const bool to_mfma = !small && (skinny(m, n, k, vec_ok, transposeA) || plan_splitk(m, n, k, SPLITK_WORKSPACE_LIMIT).chunks <= 1);
        batch_calls.push_back({a, b, c, M, N, K, alpha, beta, ldA, ldB, ldC, transposeA, transposeB, vec_ok, to_mfma});
        return 0;
    }
    scoped_record rec(fn);
    if (small) {
        dim3 blk(16, 16), grd((n + 15) / 16, (m + 15) / 16);
        hipLaunchKernelGGL(gemm_generic_kernel<float>, grd, blk, 0, current_stream, a, b, c, m, n, k,
                           transposeA ? 1L : (long)ldA, transposeA ? (long)ldA : 1L, transposeB ? 1L : (long)ldB,
                           transposeB ? (long)ldB : 1L, (long)ldC, alpha, beta);
        check(hipGetLastError(), fn);
        return 0;
    }
    if (skinny(m, n, k, vec_ok, transposeA)) {
        if (transposeB) dispatch_skinny<true>(a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta);
        else dispatch_skinny<false>(a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta);
        return 0;
    }
    // few tiles, deep reduction: K split over workgroups through a scratch buffer
    const splitk_plan plan = plan_splitk(m, n, k, SPLITK_WORKSPACE_LIMIT);
    if (plan.chunks > 1) {
        void *ws;
        if (static_scratch) {
            if (plan.scratch_bytes > STATIC_SCRATCH_BYTES) {
                fprintf(stderr, "Error at %s: %d x %d x %d needs %llu bytes of scratch for its %d K chunks of %d tiles, the static array holds %llu; "
                                "use tiramisu_hip_sgemm (which allocates) for this size\n", fn, m, n, k, (unsigned long long)plan.scratch_bytes,
                        plan.chunks, plan.tiles, (unsigned long long)STATIC_SCRATCH_BYTES);
                return 1;
            }
            ws = static_scratch_here();
        } else {
            std::lock_guard<std::mutex> g(kept_mutex);
            splitk_block &block = splitk_workspaces[here()];
            if (block.bytes < plan.scratch_bytes) {
                if (block.ptr) {
                    check(hipStreamSynchronize(current_stream), fn);
                    check(hipFree(block.ptr), fn);
                }
                check(hipMalloc(&block.ptr, plan.scratch_bytes), fn);
                block.bytes = plan.scratch_bytes;
            }
            ws = block.ptr;
        }
        const bool edge = !(vec_ok && m % SPLITK_TILE == 0 && n % SPLITK_TILE == 0 && plan.chunk % 32 == 0 && k % plan.chunk == 0);
        dispatch_splitk(plan, transposeA, transposeB, edge, a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta, vec_ok, ws);
        return 0;
    }
    const int bm = tile_for(m, n);
    const bool edge = !(vec_ok && m % bm == 0 && n % bm == 0 && k % (bm == 64 ? 32 : 16) == 0);   // K-slice of the tile
    // A is K-contiguous unless transposed; B is K-contiguous only when transposed.
    if (!transposeA && !transposeB) dispatch_edge<true, false>(edge, a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta, vec_ok);
    else if (!transposeA && transposeB) dispatch_edge<true, true>(edge, a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta, vec_ok);
    else if (transposeA && !transposeB) dispatch_edge<false, false>(edge, a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta, vec_ok);
    else dispatch_edge<false, true>(edge, a, b, c, m, n, k, ldA, ldB, ldC, alpha, beta, vec_ok);
    return 0;
}

int tiramisu_hip_sgemm(float *A, float *B, float *C, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                       uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA, uint64_t offsetB, uint64_t offsetC,
                       bool transposeA, bool transposeB) {
    return sgemm_impl(__FUNCTION__, false, A, B, C, M, N, K, alpha, beta, ldA, ldB, ldC, offsetA, offsetB, offsetC, transposeA, transposeB);
}

int tiramisu_hip_sgemm_static_scratch(float *A, float *B, float *C, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                                      uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA, uint64_t offsetB, uint64_t offsetC,
                                      bool transposeA, bool transposeB) {
    return sgemm_impl(__FUNCTION__, true, A, B, C, M, N, K, alpha, beta, ldA, ldB, ldC, offsetA, offsetB, offsetC, transposeA, transposeB);
}

int tiramisu_hip_batch_begin(void) {
    if (batch_open) return 1;          // scopes do not nest
    batch_open = true;
    batch_calls.clear();
    return 0;
}

int tiramisu_hip_batch_end(void) {
    if (!batch_open) return 1;
    batch_open = false;
    std::vector<gathered_sgemm> calls;
    calls.swap(batch_calls);
    size_t i = 0;
    while (i < calls.size()) {
        const gathered_sgemm &g = calls[i];
        size_t j = i + 1;
        if (g.to_mfma)
            while (j < calls.size() && j - i < (size_t)tgemm::BATCH_MAX && calls[j].same_shape(g)) j++;
        tgemm::sgemm_batch table;
        if (j - i > 1) {
            for (size_t q = i; q < j; q++) {
                table.A[q - i] = calls[q].a;
                table.B[q - i] = calls[q].b;
                table.C[q - i] = calls[q].c;
            }
            active_batch = &table;
            active_batch_count = (int)(j - i);
        }
        const int rc = sgemm_impl("tiramisu_hip_sgemm", false, const_cast<float *>(g.a), const_cast<float *>(g.b), g.c, g.M, g.N, g.K, g.alpha, g.beta,
                                  g.ldA, g.ldB, g.ldC, 0, 0, 0, g.tA, g.tB);
        active_batch = nullptr;
        active_batch_count = 0;
        if (rc != 0) return rc;
        i = j;
    }
    return 0;
}

void *tiramisu_hip_sgemm_workspace(void) {
    std::lock_guard<std::mutex> g(kept_mutex);
    auto it = splitk_workspaces.find(here());
    return it == splitk_workspaces.end() ? nullptr : it->second.ptr;
}

void *tiramisu_hip_kept_scratch(const void *site, uint64_t bytes, int32_t *fresh) {
    std::lock_guard<std::mutex> g(kept_mutex);
    splitk_block &block = kept_scratch[{site, here()}];
    if (fresh) *fresh = 0;
    if (block.bytes < bytes) {
        if (block.ptr) {
            check(hipStreamSynchronize(current_stream), __FUNCTION__);
            check(hipFree(block.ptr), __FUNCTION__);
        }
        check(hipMalloc(&block.ptr, bytes), __FUNCTION__);
        block.bytes = bytes;
        if (fresh) *fresh = 1;
    }
    return block.ptr;
}

uint64_t tiramisu_hip_release_cached_memory(void) {
    check(hipDeviceSynchronize(), __FUNCTION__);
    uint64_t released = 0;
    {
        std::lock_guard<std::mutex> g(kept_mutex);
        for (auto &kv : splitk_workspaces) if (kv.second.ptr) { check(hipFree(kv.second.ptr), __FUNCTION__); released += kv.second.bytes; }
        for (auto &kv : kept_scratch) if (kv.second.ptr) { check(hipFree(kv.second.ptr), __FUNCTION__); released += kv.second.bytes; }
        splitk_workspaces.clear();
        kept_scratch.clear();
    }
    std::lock_guard<std::mutex> g(pool_mutex);
    for (auto &kv : pool_free)
        for (void *q : kv.second) { check(hipFree(q), __FUNCTION__); released += kv.first; }
    pool_free.clear();
    pool_idle_bytes = 0;
    return released;
}

uint64_t tiramisu_hip_cached_memory_bytes(void) {
    uint64_t held = 0;
    {
        std::lock_guard<std::mutex> g(kept_mutex);
        for (auto &kv : splitk_workspaces) held += kv.second.bytes;
        for (auto &kv : kept_scratch) held += kv.second.bytes;
    }
    std::lock_guard<std::mutex> g(pool_mutex);
    return held + pool_idle_bytes;
}

int tiramisu_hip_dgemm(double *A, double *B, double *C, uint64_t M, uint64_t N, uint64_t K, double alpha, double beta,
                       uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA, uint64_t offsetB, uint64_t offsetC,
                       bool transposeA, bool transposeB) {
    if (ldA == 0) ldA = transposeA ? M : K;
    if (ldB == 0) ldB = transposeB ? K : N;
    if (ldC == 0) ldC = N;
    if (M == 0 || N == 0) return 0;
    scoped_record rec("tiramisu_hip_dgemm");
    if (M > 0x7fffffffull || N > 0x7fffffffull || K > 0x7fffffffull) {
        fprintf(stderr, "Error at %s: dimension exceeds 2^31-1\n", __FUNCTION__);
        exit(1);
    }
    const double *a = A + offsetA, *b = B + offsetB;
    double *c = C + offsetC;
    // element (m, k) of op(A) and (k, n) of op(B) through two strides each
    const long sam = transposeA ? 1L : (long)ldA, sak = transposeA ? (long)ldA : 1L;
    const long sbk = transposeB ? 1L : (long)ldB, sbn = transposeB ? (long)ldB : 1L;
    // 128 x 128 tiles when they give every compute unit work, else 64 x 64, and 32 x 32 for problems that would
    // leave half of the chip idle with those (the 64 x 2048 x 512 products of a recurrent cell: 128 workgroups
    // instead of 32)
    const long big = (long)((M + 127) / 128) * (long)((N + 127) / 128), medium = (long)((M + 63) / 64) * (long)((N + 63) / 64);
    if (big >= ttarget::COMPUTE_UNITS / 2) launch_dgemm<tgemm64::shape<4, 2, 2, 4>>(transposeA, transposeB, a, b, c, (int)M, (int)N, (int)K, sam, sak, sbk, sbn, (long)ldC, alpha, beta);
    else if (medium >= ttarget::COMPUTE_UNITS / 2) launch_dgemm<tgemm64::shape<2, 2, 2, 2>>(transposeA, transposeB, a, b, c, (int)M, (int)N, (int)K, sam, sak, sbk, sbn, (long)ldC, alpha, beta);
    else launch_dgemm<tgemm64::shape<1, 1, 2, 2>>(transposeA, transposeB, a, b, c, (int)M, (int)N, (int)K, sam, sak, sbk, sbn, (long)ldC, alpha, beta);
    return 0;
}

void *tiramisu_hip_module_load(const void *image, uint64_t) {
    hipModule_t m;
    check(hipModuleLoadData(&m, image), __FUNCTION__);
    return (void *)m;
}

void *tiramisu_hip_module_get_function(void *module, const char *kernel_name) {
    hipFunction_t f;
    hipError_t e = hipModuleGetFunction(&f, (hipModule_t)module, kernel_name);
    if (e != hipSuccess) {
        fprintf(stderr, "Error at %s: kernel %s: %s\n", __FUNCTION__, kernel_name, hipGetErrorString(e));
        exit(1);
    }
    {
        std::lock_guard<std::mutex> g(names_mutex);
        function_names[(void *)f] = kernel_name;
    }
    return (void *)f;
}

void *tiramisu_hip_module_get_global(void *module, const char *name, uint64_t bytes) {
    hipDeviceptr_t ptr = nullptr;
    size_t size = 0;
    check(hipModuleGetGlobal(&ptr, &size, (hipModule_t)module, name), __FUNCTION__);
    if (size < bytes) {
        fprintf(stderr, "Error at %s: symbol %s holds %zu bytes, %llu needed\n", __FUNCTION__, name, size,
                (unsigned long long)bytes);
        exit(1);
    }
    return (void *)ptr;
}

int tiramisu_hip_launch(void *function, const uint32_t grid[3], const uint32_t block[3], uint32_t dynamic_lds_bytes,
                        void **args) {
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return 0;  // empty iteration space
    if ((uint64_t)block[0] * block[1] * block[2] > (uint64_t)ttarget::MAX_THREADS_PER_WORKGROUP) {
        fprintf(stderr, "Error at %s: thread block %ux%ux%u exceeds 1024 threads\n", __FUNCTION__, block[0], block[1], block[2]);
        exit(1);
    }
    std::string nm;
    if (profiling.load()) {
        std::lock_guard<std::mutex> g(names_mutex);
        nm = function_names[function];
    }
    scoped_record rec(nm);
    check(hipModuleLaunchKernel((hipFunction_t)function, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                dynamic_lds_bytes, current_stream, args, nullptr),
          __FUNCTION__);
    return 0;
}

void tiramisu_hip_parallel_for(int32_t first, int32_t last, void (*body)(int32_t, void *), void *closure) {
    if (last < first) return;
    if (first == last || in_parallel_iteration) {
        for (int32_t i = first; i <= last; i++) body(i, closure);
        return;
    }
    static parallel_pool *pool = new parallel_pool;
    struct job { void (*body)(int32_t, void *); void *closure; } j{body, closure};
    check(hipStreamSynchronize(current_stream), __FUNCTION__);   // what the caller launched so far is complete
    pool->run(first, last, [](int32_t i, void *p) {
        in_parallel_iteration = true;
        static_cast<job *>(p)->body(i, static_cast<job *>(p)->closure);
        in_parallel_iteration = false;
    }, &j);
}

int tiramisu_hip_set_stream(void *stream) {
    current_stream = stream ? (hipStream_t)stream : hipStreamPerThread;
    return 0;
}

void *tiramisu_hip_get_stream(void) { return (void *)current_stream; }

void *tiramisu_hip_stream_create(void) {
    hipStream_t s;
    check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), __FUNCTION__);   // default priority
    return (void *)s;
}

int tiramisu_hip_stream_destroy(void *stream) {
    if (!stream) return 0;
    check(hipStreamSynchronize((hipStream_t)stream), __FUNCTION__);
    if (current_stream == (hipStream_t)stream) current_stream = hipStreamPerThread;
    check(hipStreamDestroy((hipStream_t)stream), __FUNCTION__);
    return 0;
}

void *tiramisu_hip_event_create(void) {
    hipEvent_t e;
    check(hipEventCreate(&e), __FUNCTION__);
    return (void *)e;
}

int tiramisu_hip_event_record(void *event) {
    check(hipEventRecord((hipEvent_t)event, current_stream), __FUNCTION__);
    return 0;
}

float tiramisu_hip_event_elapsed_ms(void *start, void *stop) {
    float ms = 0.f;
    check(hipEventSynchronize((hipEvent_t)stop), __FUNCTION__);
    check(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop), __FUNCTION__);
    return ms;
}

int tiramisu_hip_event_destroy(void *event) {
    check(hipEventDestroy((hipEvent_t)event), __FUNCTION__);
    return 0;
}

int tiramisu_hip_profile_start(void) {
    std::lock_guard<std::mutex> g(records_mutex);
    for (auto &r : records) {
        hipEventDestroy(r.start);
        hipEventDestroy(r.stop);
    }
    records.clear();
    profiling = true;
    return 0;
}

int tiramisu_hip_profile_stop(void) {
    profiling = false;
    std::lock_guard<std::mutex> g(records_mutex);
    for (auto &r : records) {
        check(hipEventSynchronize(r.stop), __FUNCTION__);
        check(hipEventElapsedTime(&r.ms, r.start, r.stop), __FUNCTION__);
    }
    return (int)records.size();
}

const char *tiramisu_hip_profile_name(int record) {
    return (record >= 0 && record < (int)records.size()) ? records[record].name.c_str() : "";
}

float tiramisu_hip_profile_ms(int record) {
    return (record >= 0 && record < (int)records.size()) ? records[record].ms : 0.f;
}

int tiramisu_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

}  // extern "C"
