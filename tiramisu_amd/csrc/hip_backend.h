// The HIP (gfx950) back-end: shared declarations of the kernel emitters and the host-glue
// emitter.  Replaces the reference's CUDA printer (src/tiramisu_codegen_cuda.cpp,
// include/tiramisu/cuda_ast.h) and the GPU half of its Halide host path
// (src/tiramisu_codegen_halide.cpp:2014-2040, :1773-1862, :2576-2607).
#ifndef TIRAMISU_AMD_HIP_BACKEND_H
#define TIRAMISU_AMD_HIP_BACKEND_H
#include <set>
#include <string>
#include <vector>

#include <tiramisu/core.h>

#include "c_print.h"
#include "lir.h"

namespace tiramisu {
namespace hipgen {

struct kernel_param {
    bool is_buffer;
    std::string name;
    primitive_t type;  // element type for buffers
};

/** One device kernel plus everything the host needs to launch it.  grid/block hold host-side
  * expression texts, x first. */
struct kernel {
    std::string name;
    std::string source;                 // text of the kernel (and its private helpers)
    std::vector<kernel_param> params;   // launch order: scalars sorted by name, then buffers
    std::string grid[3] = {"1", "1", "1"};
    std::string block[3] = {"1", "1", "1"};
    std::string lds_bytes = "0";
    std::string batch_first;            // not empty: the launch site declares `_batch_first` with this value (a parameter)
    std::string how;                    // "generic", "mfma-contraction", "stencil", ...
    /** Host buffers that the kernel names (only with implicit copies): the launch site gives it
      * device copies of them, copied in before the launch and, when written, back after it. */
    struct host_mirror { std::string name, ctype, bytes; bool written; };
    std::vector<host_mirror> host_mirrors;
};

/** A launch sequence that replaces one GPU-tagged loop nest. */
struct launch_plan {
    std::vector<kernel> kernels;
    /** Host statements run instead of a plain launch of kernels[0] (empty = launch each once). */
    std::string host_code;
};

struct context {
    function *f = nullptr;
    lir::program *prog = nullptr;
    std::vector<kernel> kernels;        // all kernels of the function, in emission order
    std::string includes;               // extra text at the top of the kernel file
    std::set<std::string> include_once;
    std::set<std::string> constant_buffers;   // buffers living in the code object's constant memory
    std::vector<std::string> host_iterators;  // iterators of the host loops around the nest being emitted
    int next_kernel_id();
    /** The number the next kernel gets; set_next_kernel_id() takes numbers back when an attempt
      * that already named kernels is abandoned. */
    static int peek_next_kernel_id();
    static void set_next_kernel_id(int id);
};

/** What the contraction emitter may fold into its kernel beyond the nest itself.
  *  * consumer: the GPU-mapped nest that follows the contraction in the same host loop body.  When
  *    its statements are point-wise over (row, unit) and read the contraction's result only at the
  *    row's own columns `unit + q * units` (q = 0, 1, ...: column groups, e.g. the four gates of a
  *    recurrent cell), they run in the contraction kernel, on the tile that the workgroup has just
  *    finished: columns are dealt to workgroups so that a tile holds all groups of its units.
  *  * batch_iterator: a host loop tagged parallel around the nest; its iterations become
  *    gridDim.z of one launch instead of launches of their own. */
struct fusion_request {
    lir::node_ptr consumer;
    std::string batch_iterator;
    expr batch_first, batch_last;
};

/** Schedule-faithful kernel: one thread per (block-iterator, thread-iterator) point, untagged
  * inner loops serial in the thread (reference: tiramisu_codegen_cuda.cpp:239-326, :549-707). */
kernel emit_generic_kernel(context &ctx, const lir::node_ptr &root);
/** The same with the iterations of a host loop tagged parallel around the nest as gridDim.z of one launch: the
  * kernel recomputes the loop's iterator from blockIdx.z (fusion_request's batch_* fields; its consumer is not
  * used).  \p ok is false, and nothing is kept, when the nest's own grid already uses z or its extents involve the
  * iterator. */
kernel emit_generic_kernel_batched(context &ctx, const lir::node_ptr &root, const fusion_request &batch, bool &ok);

/** Pattern-directed emitters.  Each returns false when the nest is not provably of its kind, in
  * which case the generic emitter is used. */
bool emit_contraction(context &ctx, const lir::node_ptr &root, launch_plan &plan, const fusion_request *fuse = nullptr);
bool emit_stencil(context &ctx, const lir::node_ptr &root, const lir::node_ptr &time_loop, launch_plan &plan);

/** Directory of the kernel headers that emitted code includes (TIRAMISU_AMD_KERNEL_DIR overrides the
  * one compiled in), and the helper that adds an #include line to the kernel file once. */
std::string kernel_dir();
std::string include_dir();
void add_include_once(context &ctx, const std::string &line);

/** Text of the launch of \p k with the argument list taken from host variables of the same names. */
std::string launch_text(const kernel &k, const std::string &indent);

}  // namespace hipgen
}  // namespace tiramisu
#endif
