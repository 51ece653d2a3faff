// Front-end of the Tiramisu embedded compiler, re-provided without Halide on top of isl:
// function / buffer / computation / input / constant, the scheduling commands, the GPU
// mapping commands and codegen().  Interface follows include/tiramisu/core.h of the
// reference (function :189, buffer :1424, computation :1863, input :4952,
// constant :5212); the implementation is new and lowers to HIP for gfx950.
#ifndef TIRAMISU_AMD_CORE_H
#define TIRAMISU_AMD_CORE_H
#include <cassert>
#include <cmath>
#include <array>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include <tiramisu/debug.h>
#include <tiramisu/expr.h>
#include <tiramisu/type.h>

struct isl_ctx;
struct isl_set;
struct isl_map;
struct isl_ast_node;
struct isl_union_map;

namespace tiramisu {

class function;
class computation;
class buffer;
class constant;
class input;
class view;
class block;
namespace lir { struct program; }

/** Start a new implicit function called \p name (reference: tiramisu_core.cpp:60-70). */
void init(std::string name);
void init();

/** Generate code for the implicit function.  \p arguments are the buffers of the generated
  * function's signature, in order.  \p gen_gpu true selects the GPU back-end (HIP, gfx950);
  * false selects the CPU back-end, which must be linked separately (it lives with the
  * parity oracle and is not part of the GPU product library).
  * Reference: tiramisu_core.cpp:88-98, tiramisu_function.cpp:2540-2602. */
void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename,
             const bool gen_gpu = false);
void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename,
             const hardware_architecture_t gen_architecture_flag);

/** function::set_backend_option on the implicit function. */
void set_backend_option(const std::string &name, const std::string &value);
void set_backend_option(const std::string &name, long value);
/** Lets whoever runs a generator program choose back-end options: every "--backend-option name=value" (or
  * "--backend-option=name=value") among the arguments becomes an option of every function that tiramisu::init
  * creates afterwards; the program's own set_backend_option calls still override them.  Other arguments are
  * left alone; returns the number of options taken.  Call it first thing in main(argc, argv). */
int backend_options_from_command_line(int argc, char **argv);
/** The option of the function whose code is being generated (of the implicit function outside code
  * generation); plain getenv when there is no function at all.  For the back-end's own sources. */
const char *backend_option(const char *env_name);

/** The same calls on the implicit function (reference: core.h:139-181). */
void perform_full_dependency_analysis();
bool check_legality_of_function();
void prepare_schedules_for_legality_checks(bool reset_static_dimesion = false);
bool loop_parallelization_is_legal(var i, std::vector<computation *> fused_computations);
bool loop_unrolling_is_legal(var i, std::vector<computation *> fused_computations);
bool loop_vectorization_is_legal(var i, std::vector<computation *> fused_computations);

/** GPU memory spaces of a buffer (reference: cuda_ast.h:180-188). */
enum class memory_location { host, global, shared, local, constant, reg };

/** A code-generation back-end: turns the lowered loop program of a function into an
  * artefact on disk.  Back-ends register themselves by architecture. */
class backend {
public:
    virtual ~backend() {}
    virtual void generate(function &f, lir::program &prog, const std::string &obj_filename) = 0;
    static void register_backend(hardware_architecture_t arch, backend *b);
    static backend *find(hardware_architecture_t arch);
};

class function {
    friend class computation;
    friend class buffer;
    friend class constant;
    friend class input;

    std::string name;
    isl_ctx *ctx = nullptr;
    std::vector<computation *> body;          // in declaration order
    std::vector<computation *> invariants;    // function-wide constants
    std::map<std::string, buffer *> buffers_list;
    std::vector<buffer *> function_arguments;
    isl_set *context_set = nullptr;
    isl_ast_node *ast = nullptr;
    std::unique_ptr<lir::program> lowered;
    std::vector<std::string> iterator_names;

public:
    // (computation name, level) tags
    std::set<std::pair<std::string, int>> parallel_dimensions;
    std::map<std::pair<std::string, int>, int> vector_dimensions;   // -> vector length
    std::map<std::pair<std::string, int>, int> unroll_dimensions;   // -> factor (0 = full)
    std::set<std::pair<std::string, int>> distributed_dimensions;
    /** (computation name, (l0,l1,l2)) with -1 for unused levels, outermost first
      * (reference: core.h:340-346). */
    std::vector<std::pair<std::string, std::tuple<int, int, int>>> gpu_block_dimensions;
    std::vector<std::pair<std::string, std::tuple<int, int, int>>> gpu_thread_dimensions;

    /** Ordering graph: sched_graph[a][b] = level means "b right after a, fused down to level". */
    std::unordered_map<computation *, std::unordered_map<computation *, int>> sched_graph;
    std::unordered_map<computation *, std::unordered_map<computation *, int>> sched_graph_reversed;
    std::set<computation *> starting_computations;
    bool use_low_level_scheduling_commands = false;

    std::map<std::string, std::string> backend_options;                          // set_backend_option
    mutable std::vector<std::array<std::string, 3>> consulted_options;          // backend_option

    explicit function(std::string name);
    ~function();

    const std::string &get_name() const { return name; }
    isl_ctx *get_isl_ctx() const { return ctx; }
    const std::vector<computation *> &get_computations() const { return body; }
    std::vector<computation *> get_computation_by_name(std::string nm) const;
    const std::vector<computation *> &get_invariants() const { return invariants; }
    std::vector<std::string> get_invariant_names() const;
    const std::map<std::string, buffer *> &get_buffers() const { return buffers_list; }
    const std::vector<buffer *> &get_arguments() const { return function_arguments; }
    void add_computation(computation *c);
    void add_invariant(constant *c);
    void add_buffer(std::pair<std::string, buffer *> b);
    void add_context_constraints(std::string constraints);
    void set_context_set(const std::string &s) { add_context_constraints(s); }
    isl_set *get_program_context() const { return context_set; }
    void set_iterator_names(const std::vector<std::string> &names) { iterator_names = names; }
    const std::vector<std::string> &get_iterator_names() const { return iterator_names; }

    void add_parallel_dimension(std::string comp, int level);
    void add_vector_dimension(std::string comp, int level, int length);
    void add_unroll_dimension(std::string comp, int level, int factor);
    void add_gpu_block_dimensions(std::string comp, int l0, int l1 = -1, int l2 = -1);
    void add_gpu_thread_dimensions(std::string comp, int l0, int l1 = -1, int l2 = -1);
    bool should_parallelize(const std::string &comp, int level) const;
    int vector_length(const std::string &comp, int level) const;     // 0 if untagged
    bool should_unroll(const std::string &comp, int level) const;
    /** 0..2 = block z..x / thread index position in its tuple, -1 if the level is not mapped. */
    int gpu_block_position(const std::string &comp, int level) const;
    int gpu_thread_position(const std::string &comp, int level) const;

    // ---- the code generation pipeline (reference: tiramisu_function.cpp:2540-2562) ----
    /** CPU buffer name -> the GPU buffer declared as its counterpart (the last argument of the
      * buffer constructor); reference: core.h:903-911. */
    std::map<std::string, buffer *> mapping;
    const std::map<std::string, buffer *> &get_mapping() const { return mapping; }
    void add_mapping(std::pair<std::string, buffer *> p) { mapping.insert(p); }
    /** First / last computation of the ordering chain (reference: tiramisu_function.cpp:1141-1165). */
    computation *get_first_cpt();
    computation *get_last_cpt();
    /** Insert the host-to-device copies of mapped input buffers before \p c1 and the device-to-host
      * copies of mapped output buffers after \p c2 (reference: tiramisu_function.cpp:379-435).
      * Called by codegen() for a GPU target when the function has mapped buffers. */
    void Automatic_communication(computation *c1, computation *c2);

    void set_arguments(const std::vector<buffer *> &buffer_vec);
    /** Turn the ordering graph into static schedule dimensions (reference :2231-2295). */
    void gen_ordering_schedules();
    /** Pad all schedules to the same number of dimensions (reference :1774-1794). */
    void align_schedules();
    void gen_time_space_domain();
    /** Build the isl AST and lower it to the loop program shared by all back-ends. */
    void gen_isl_ast();
    isl_ast_node *get_isl_ast() const { return ast; }
    lir::program &get_lowered_program();
    /** Stages of the reference pipeline that existing programs call by hand; in this build
      * gen_cuda_stmt selects the GPU back-end and gen_halide_obj runs it. */
    void gen_cuda_stmt() { hand_driven_gpu = true; }
    void gen_halide_stmt() {}
    void gen_halide_obj(const std::string &obj_file_name);
    void gen_c_code() const;
    void dump_halide_stmt() const {}
    void dump(bool exhaustive = false) const;
    void dump_schedule() const;
    void dump_sched_graph();
    /** Gives every computation that stores somewhere and has no buffer yet a buffer shaped after its
      * iteration domain (largest index + 1 per dimension) and maps it one to one: computations that no
      * other computation reads become outputs, unscheduled ones (read only) inputs, the rest temporaries
      * (reference: tiramisu_function.cpp:1458-1511, tiramisu_core.cpp:2268-2335). */
    void allocate_and_map_buffers_automatically();
    void dump_dep_graph();
    /** Infer iteration domains from consumers: starting from the computations that nothing reads, a
      * computation's domain becomes what its consumers read of it (joined with the domain it was declared
      * with, unless that was unbounded); computations with several definitions keep theirs
      * (reference: tiramisu_function.cpp:624-747). */
    void compute_bounds();
    /** Computations that no other computation reads (reference: tiramisu_function.cpp:503-615). */
    std::vector<computation *> get_live_out_computations();
    /** Print the iteration domains / the time-space domains (domain mapped through the schedule) of all
      * computations (reference: core.h:1071-1109). */
    void dump_iteration_domain() const;
    void dump_time_processor_domain() const;
    void dump_trimmed_time_processor_domain() const { dump_time_processor_domain(); }
    constant *get_invariant_by_name(std::string str) const;

    // ---- dependence analysis and legality of schedules
    //      (reference: tiramisu_function.cpp:165-357, :2618-3047, :3091-3660; core.h:1236-1330)
    /** Results of perform_full_dependency_analysis(), each { source instance -> [sink instance -> buffer cell] }
      * over the iteration domains: the last write before every read, the reads before every write that no write
      * between them hides, the last write before every write; then { instance -> cell } for the reads that see no
      * write of this function and for the writes that nothing overwrites. */
    isl_union_map *dep_read_after_write = nullptr;
    isl_union_map *dep_write_after_read = nullptr;
    isl_union_map *dep_write_after_write = nullptr;
    isl_union_map *live_in_access = nullptr;
    isl_union_map *live_out_access = nullptr;
    /** Dataflow analysis of the program as scheduled at the time of the call: call it once every computation has
      * its buffer (store_in) and before the schedule commands whose legality is in question. */
    void perform_full_dependency_analysis();
    void calculate_dep_flow(bool global_memory_only = false);
    /** Aligns and orders the schedules (after/then/between) so that they can be compared; \p reset_static_dimesion
      * first clears the ordering an earlier call left in the static dimensions. */
    void prepare_schedules_for_legality_checks(bool reset_static_dimesion = false);
    void reset_all_static_dims_to_zero();
    /** True when, under the present schedules, the source of every dependence is executed strictly before its
      * sink; the second form looks only at dependences between the computations given. */
    bool check_legality_for_function();
    bool check_partial_legality_in_function(std::vector<computation *> involved_computations);
    /** True when no dependence between the computations given (fused in that loop) is carried by loop \p i. */
    bool loop_parallelization_is_legal(var i, std::vector<computation *> fused_computations);
    bool loop_parallelization_is_legal(int parallel_dim, std::vector<computation *> fused_computations);
    /** True when the bounds of loop \p i are one affine expression of the outer loops each (no min/max). */
    bool loop_unrolling_is_legal(var i, std::vector<computation *> fused_computations);
    bool loop_vectorization_is_legal(var i, std::vector<computation *> fused_computations);
    /** The smallest non-negative shifts of \p current along \p vars_subjected_to_shifting (lexicographically,
      * outer loop first) that make every dependence between it and \p previous_computations -- the computations
      * fused before it -- legal; one (var, shift) per variable, or nothing when no shift does or a dependence
      * distance is not constant up to the innermost of the variables. */
    std::vector<std::tuple<var, int>> correcting_loop_fusion_with_shifting(std::vector<computation *> previous_computations,
                                                                          computation &current,
                                                                          std::vector<var> vars_subjected_to_shifting);
    /** The race check of the GPU mapping: one line for every loop tagged as a block or thread dimension that, in
      * the program as scheduled now, carries a dependence through global memory (what goes through LDS is ordered
      * by the program's barriers and is left out).  codegen() for the GPU calls it and stops on a finding when
      * the environment variable TIRAMISU_HIP_CHECK_MAPPED_LOOPS is set. */
    std::vector<std::string> gpu_mapped_loops_that_carry_dependences();
    /** The five results of the analysis, one "name: relation" line each. */
    std::string dependences_as_text() const;
    /** Skewings of two consecutive loops, from the distances of the dependences among \p fused_computations at
      * those loops (reference: core.h:1325-1384): pairs (a, b) for computation::skew(i, j, a, b) after which the outer
      * loop is parallel (first vector, at most one), the inner loop is parallel (second: the \p nb_parallel smallest
      * with b > 0, then with b < 0), or some dependence stays inside one iteration of the outer loop (third: one
      * with b > 0, one with b < 0; the inner loop may then have to be reversed).  Empty vectors when there is no
      * dependence at these loops or no skewing with coefficients up to 8 does it. */
    std::tuple<std::vector<std::pair<int, int>>, std::vector<std::pair<int, int>>, std::vector<std::pair<int, int>>>
    skewing_local_solver(std::vector<computation *> fused_computations, var outer_variable, var inner_variable, int nb_parallel);
    /** The same with all four coefficients (alpha, beta, gamma, sigma) of computation::skew, chosen so that every
      * distance has non-negative components afterwards (both loops can then be tiled); the third vector holds
      * the skewing of the inner loop alone, (1, 0, gamma, 1). */
    std::tuple<std::vector<std::tuple<int, int, int, int>>, std::vector<std::tuple<int, int, int, int>>, std::vector<std::tuple<int, int, int, int>>>
    skewing_local_solver_positive(std::vector<computation *> fused_computations, var outer_variable, var inner_variable, int nb_parallel);
    /** Every dependence as { source instance -> sink instance }. */
    isl_union_map *get_statement_dependences() const;
    void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename,
                 const hardware_architecture_t arch);
    void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename,
                 const bool gen_gpu = false);
    int get_max_schedules_range_dim() const;
    std::string generate_new_name(const std::string &prefix);
    const std::vector<std::string> &get_codegen_log() const { return codegen_log; }
    void log(const std::string &s) { codegen_log.push_back(s); }

    // ---- options of the code-generation back-end (no counterpart in the reference, whose CUDA back-end has none)
    /** Sets an option of the back-end for this function: tile shapes, steps fused per stencil launch, which
      * emitters may take a nest, and so on.  An option is named after its environment variable without the
      * TIRAMISU_ prefix, in lower case: "stencil_rows", "mfma_tile", "no_single_step_stencil"; switches take
      * "1".  The environment variable, when set, overrides the program's value (so a run can still be
      * steered from outside); the manifest written beside the object lists every option that code generation
      * found set, with its value and where it came from.  An empty value removes the option. */
    void set_backend_option(const std::string &name, const std::string &value);
    void set_backend_option(const std::string &name, long value) { set_backend_option(name, std::to_string(value)); }
    void clear_backend_options() { backend_options.clear(); }
    const std::map<std::string, std::string> &get_backend_options() const { return backend_options; }
    /** The value of the option whose environment variable is \p env_name ("TIRAMISU_STENCIL_ROWS"): the
      * environment's, else the program's, else null.  Remembers what it found for the manifest. */
    const char *backend_option(const char *env_name) const;
    /** (option, value, "environment" | "program") of every option looked up and found set since the last
      * clear_consulted_backend_options(). */
    const std::vector<std::array<std::string, 3>> &consulted_backend_options() const { return consulted_options; }
    void clear_consulted_backend_options() const { consulted_options.clear(); }

    /** True when GPU-mapped loops are generated without gen_cuda_stmt() -- the route that, in the
      * reference, hands the loops to Halide's own GPU target, which moves buffers between host and
      * device by itself: kernels may then name host buffers, and the host glue copies them around
      * each launch. */
    bool copies_host_buffers_implicitly() const { return implicit_gpu_copies; }

private:
    bool hand_driven_gpu = false;
    bool implicit_gpu_copies = false;
    int name_counter = 0;
    std::vector<std::string> codegen_log;
};

class buffer {
    friend class computation;
    friend class function;
    std::string name;
    std::vector<expr> dim_sizes;  // outermost first; last dimension is contiguous
    primitive_t type;
    argument_t argtype;
    function *fct;
    bool allocated = false;
    bool auto_allocate = true;
    bool auto_deallocate = true;

public:
    memory_location location = memory_location::host;
    /** Whether codegen() inserts the copies between this GPU buffer and its CPU counterpart
      * (reference: core.h:1467-1470). */
    bool automatic_gpu_copy = true;
    bool get_automatic_gpu_copy() const { return automatic_gpu_copy; }
    void set_automatic_gpu_copy(bool v) { automatic_gpu_copy = v; }

    /** Reference: tiramisu_core.cpp:6762-6781. */
    buffer(std::string name, std::vector<expr> dim_sizes, primitive_t type, argument_t argt,
           function *fct = global::get_implicit_function(), std::string corr = "");

    const std::string &get_name() const { return name; }
    int get_n_dims() const { return (int)dim_sizes.size(); }
    primitive_t get_elements_type() const { return type; }
    const std::vector<expr> &get_dim_sizes() const { return dim_sizes; }
    argument_t get_argument_type() const { return argtype; }
    void set_argument_type(argument_t t) { argtype = t; }
    memory_location get_location() const { return location; }
    bool get_auto_allocate() const { return auto_allocate; }
    bool get_auto_deallocate() const { return auto_deallocate; }
    void set_auto_allocate(bool v) { auto_allocate = v; }
    void set_auto_deallocate(bool v) { auto_deallocate = v; }
    bool has_constant_extents() const;
    function *get_function() const { return fct; }
    /** Reference: tiramisu_core.cpp:8159-8167. */
    void set_dim_size(int dim, int size);

    /** Memory-space tags (reference: tiramisu_core.cpp:8913-8936). */
    void tag_gpu_global() { location = memory_location::global; }
    void tag_gpu_shared() { location = memory_location::shared; auto_allocate = false; }
    void tag_gpu_local() { location = memory_location::local; auto_allocate = false; }
    void tag_gpu_register();
    void tag_gpu_constant() { location = memory_location::constant; }

    /** Allocate (resp. free) this buffer right before (after) \p C at loop level \p level
      * (reference: tiramisu_core.cpp:1479-1631). */
    computation *allocate_at(computation &C, var level);
    computation *allocate_at(computation &C, int level);
    computation *deallocate_at(computation &C, var level);
    computation *deallocate_at(computation &C, int level);
    void dump(bool exhaustive) const;
};

class computation {
    friend class function;
    friend class buffer;
    friend class input;
    friend class constant;
    friend class block;

protected:
    std::string name;
    function *fct = nullptr;
    isl_ctx *ctx = nullptr;
    isl_set *iteration_domain = nullptr;
    isl_map *schedule = nullptr;          // domain -> [dup, s0, d0, s1, ..., d(n-1), sn]
    isl_map *access = nullptr;            // domain -> buffer
    isl_set *time_space_domain = nullptr;
    std::vector<std::string> level_names; // names of the dynamic dimensions, outermost first
    std::vector<std::string> iterator_names_;  // names of the iteration-domain dimensions
    expr expression;
    expr predicate;
    primitive_t data_type = p_none;
    bool schedule_this = true;
    bool is_let = false;
    computation *first_definition = nullptr;     // set for an update
    std::vector<computation *> updates;          // of a first definition
    bool inline_ = false;
    buffer *automatically_allocated_buffer = nullptr;
    std::vector<std::pair<std::string, expr>> associated_let_stmts;
    std::vector<var> declared_vars;

public:
    /** One LDS tile installed by cache_shared(): the input it caches, the tile's shape and origin,
      * and the computations that declare, fill and fence it. */
    struct shared_cache {
        std::string input, access;
        std::vector<int> shape;
        std::vector<expr> offsets;
        int copy_level = -1;
        std::vector<computation *> apparatus;
    };

protected:
    expr uncached_expression;             // expression before cache_shared() redirected loads to LDS tiles
    std::vector<shared_cache> shared_caches;
    computation *cache_consumer = nullptr;  // set on the computations that cache_shared() creates

    computation() {}
    void init_computation(std::string iteration_space_str, function *f, const expr &e,
                          bool schedule_this_computation, primitive_t t);
    std::string construct_iteration_domain(const std::string &nm, const std::vector<var> &vars);
    void set_identity_schedule();
    int dynamic_pos(int level) const { return 2 * level + 2; }
    int static_pos(int level_plus_one) const { return 2 * level_plus_one + 1; }
    void apply_on_range(const std::string &transformation);
    void assert_names_not_assigned(const std::vector<std::string> &names) const;
    void separate_and_split(int level, int factor, const std::string &outer,
                            const std::string &inner, bool &split_applied);
    computation *copy_as(const std::string &new_name);
    void separate_by_text(int dim, const std::string &bound_text, const std::string &params);
    std::vector<computation *> duplicates;

public:
    static const var root;
    static constexpr int root_dimension = -1;

    /** Low-level constructor from an isl set string such as
      * "[N]->{S[i,j]: 0<=i<N and 0<=j<N}" (reference: core.h:3148-3152). */
    computation(std::string iteration_domain, expr e, bool schedule_this_computation,
                primitive_t t, function *fct);
    computation(std::string name, std::vector<var> iterator_variables, expr e,
                bool schedule_this_computation);
    computation(std::vector<var> iterator_variables, expr e);
    computation(std::string name, std::vector<var> iterator_variables, expr e);
    computation(std::vector<var> iterator_variables, expr predicate, expr e);
    computation(std::string name, std::vector<var> iterator_variables, expr predicate, expr e);
    computation(std::vector<var> iterator_variables, expr e, bool schedule_this_computation);
    computation(std::string name, std::vector<var> iterator_variables, primitive_t t)
        : computation(name, iterator_variables, expr(t)) {}
    computation(std::vector<var> iterator_variables, primitive_t t)
        : computation(iterator_variables, expr(t)) {}
    virtual ~computation();

    // ---- queries ----
    const std::string &get_name() const { return name; }
    function *get_function() const { return fct; }
    isl_ctx *get_ctx() const { return ctx; }
    isl_set *get_iteration_domain() const { return iteration_domain; }
    isl_map *get_schedule() const { return schedule; }
    isl_map *get_access_relation() const { return access; }
    isl_set *get_time_space_domain() const { return time_space_domain; }
    const expr &get_expr() const { return expression; }
    const expr &get_predicate() const { return predicate; }
    primitive_t get_data_type() const { return data_type; }
    int get_iteration_domain_dimensions_number() const;
    /** Lowest and highest value of iteration-domain dimension \p dim among the iterations that this computation
      * executes (its iteration domain restricted by its schedule: separated pieces and duplicates execute a
      * part); false when there is none or the range is not a pair of constants. */
    bool executed_range(int dim, long &lowest, long &highest) const;
    int get_loop_levels_number() const { return (int)level_names.size(); }
    const std::vector<std::string> &get_loop_level_names() const { return level_names; }
    const std::vector<std::string> &get_iteration_domain_dimension_names() const { return iterator_names_; }
    bool should_schedule_this_computation() const { return schedule_this; }
    bool is_let_stmt() const { return is_let; }
    /** Expression as written, before cache_shared() redirected loads (undefined when it never did). */
    const expr &get_uncached_expr() const { return uncached_expression; }
    const std::vector<shared_cache> &get_shared_caches() const { return shared_caches; }
    /** The computation whose loads this one serves, when cache_shared() created it. */
    computation *get_cache_consumer() const { return cache_consumer; }
    /** True when, under the current schedule, every LDS tile of this computation is proven to
      * hold exactly the elements that the computation reads through it in each iteration of
      * the copy level: reading the tile then equals reading the cached input directly. */
    bool shared_caches_cover_reads() const;
    bool is_inline_computation() const { return inline_; }
    bool has_accesses() const;
    buffer *get_buffer() const;
    buffer *get_automatically_allocated_buffer() const { return automatically_allocated_buffer; }

    /** Further definitions of this computation over other parts of its domain ("updates": C[0] = ...,
      * then C[i] = f(C[i-1]) for i >= 1).  Each is a computation of its own for scheduling and data
      * mapping, reached with get_update(k) (0 is this computation); accesses C(...) in expressions read
      * through the first definition's mapping, so all definitions are expected to store in one buffer
      * (reference: core.h:3236-3262, tiramisu_core.cpp:254-273; internally a definition is named
      * _<name>_update_<k>). */
    /** Gives this computation a temporary buffer of its whole size, allocated inside the loop nest of
      * \p comp at loop level \p L0, right before \p comp there (reference: tiramisu_core.cpp:1138-1171);
      * returns the allocation. */
    computation *store_at(computation &comp, var L0);
    void add_definitions(std::string iteration_domain, expr e, bool schedule_this_computation, primitive_t t, function *fct);
    computation &get_update(int index);
    computation *get_first_definition() { return first_definition ? first_definition : this; }
    computation &get_last_update() { return updates.empty() ? *this : *updates.back(); }
    bool is_first_definition() const { return first_definition == nullptr; }
    const std::vector<computation *> &get_updates() const { return updates; }
    buffer *auto_buffer() const { return automatically_allocated_buffer; }
    const std::vector<std::pair<std::string, expr>> &get_associated_let_stmts() const { return associated_let_stmts; }
    int get_loop_level_number_from_dimension_name(std::string dim_name) const {
        return get_loop_level_numbers_from_dimension_names({dim_name})[0];
    }
    /** Look dimension names up in the schedule range; "root" gives -1
      * (reference: tiramisu_core.cpp:2725-2770). */
    std::vector<int> get_loop_level_numbers_from_dimension_names(const std::vector<std::string> &names) const;
    void dump_iteration_domain() const;
    void dump_schedule() const;
    void dump() const;

    // ---- definition ----
    void set_expression(const expr &e);
    void add_predicate(expr p) { predicate = p; }
    void add_associated_let_stmt(std::string nm, expr e) { associated_let_stmts.push_back({nm, e}); }
    void set_inline(bool is_inline = true) { inline_ = is_inline; }
    void set_access(std::string access_str);
    void set_access(isl_map *acc);
    void store_in(buffer *buff);
    void store_in(buffer *buff, std::vector<expr> iterators);
    void store_in(std::vector<expr> mapping, std::vector<expr> sizes);
    void allocate_and_map_buffer_automatically(argument_t type = a_temporary);
    void unschedule_this_computation() { schedule_this = false; }

    template <typename... Args> expr operator()(Args... args) {
        std::vector<expr> idx{expr(args)...};
        return make_access(idx);
    }
    expr make_access(const std::vector<expr> &idx);
    operator expr();

    // ---- ordering (reference: tiramisu_core.cpp:2352-2496) ----
    void after(computation &comp, var iterator);
    void after(computation &comp, int level);
    void after_low_level(computation &comp, int level);
    void before(computation &consumer, var L);
    void before(computation &consumer, int L);
    void between(computation &before_comp, var before_l, computation &after_comp, var after_l);
    void between(computation &before_comp, int before_l, computation &after_comp, int after_l);
    computation &then(computation &next_computation, var L = computation::root);
    computation &then(computation &next_computation, int L);
    void fuse_after(var lev, computation &comp) { after(comp, lev); }
    computation *get_predecessor();
    computation *get_successor();

    // ---- loop transformations ----
    virtual void split(var L0, int sizeX);
    virtual void split(var L0, int sizeX, var L0_outer, var L0_inner);
    virtual void split(int L0, int sizeX);
    virtual void tile(var L0, var L1, int sizeX, int sizeY);
    virtual void tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer,
                      var L0_inner, var L1_inner);
    virtual void tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ);
    virtual void tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer,
                      var L1_outer, var L2_outer, var L0_inner, var L1_inner, var L2_inner);
    virtual void tile(int L0, int L1, int sizeX, int sizeY);
    virtual void tile(int L0, int L1, int L2, int sizeX, int sizeY, int sizeZ);
    virtual void interchange(var L0, var L1);
    virtual void interchange(int L0, int L1);
    virtual void shift(var L0, int n);
    virtual void shift(int L0, int n);
    virtual void skew(var i, var j, int factor, var ni, var nj);
    virtual void skew(var i, var j, int factor);
    virtual void skew(int i, int j, int factor);
    /** Generalised skewing of two consecutive loops (reference: tiramisu_core.cpp:4305-4531, :4533-4560):
      * i' = a i + b j, and j' = gamma i + sigma j with a sigma - gamma b = 1 -- gamma and sigma given,
      * or found as the reference finds them (a, b reduced by their gcd first). */
    virtual void skew(var i, var j, int a, int b, var ni, var nj);
    virtual void skew(int i, int j, int a, int b);
    virtual void skew(var i, var j, int alpha, int beta, int gamma, int sigma, var ni, var nj);
    virtual void skew(int i, int j, int alpha, int beta, int gamma, int sigma);
    /** Skewing of three / four consecutive loops by one factor: j' = f i + j, k' = f i + k (, l' = f i + l)
      * (reference: tiramisu_core.cpp:3813-3972, :3974-4160). */
    virtual void skew(var i, var j, var k, int factor, var ni, var nj, var nk);
    virtual void skew(var i, var j, var k, var l, int factor, var ni, var nj, var nk, var nl);
    virtual void skew(var i, var j, var k, int factor);
    virtual void skew(var i, var j, var k, var l, int factor);
    virtual void skew(int i, int j, int k, int l, int factor);
    /** Legality of the present schedules for the dependences from this computation to \p second
      * (reference: tiramisu_core.cpp:4695-4904); after function::perform_full_dependency_analysis(). */
    virtual bool involved_subset_of_dependencies_is_legal(computation *second);
    /** True when the bounds of loop \p l are single affine expressions of the loops around it
      * (reference: tiramisu_core.cpp:4906-5011). */
    virtual bool unrolling_is_legal(var l);
    virtual void loop_reversal(var old_var, var new_var);
    virtual void loop_reversal(int i);
    virtual void parallelize(var L);
    virtual void vectorize(var L, int v);
    virtual void vectorize(var L, int v, var L_outer, var L_inner);
    virtual void unroll(var L, int fac);
    virtual void unroll(var L, int fac, var L_outer, var L_inner);
    void tag_parallel_level(var L);
    void tag_parallel_level(int L);
    void tag_vector_level(var L, int len);
    void tag_vector_level(int L, int len);
    void tag_unroll_level(var L);
    void tag_unroll_level(var L, int F);
    void tag_unroll_level(int L);
    void tag_unroll_level(int L, int F);
    // ---- separation, redundant computation, storage folding ----
    /** Cut this computation in two at loop level \p dim: it keeps the iterations below
      * lower_bound + v * floor(N / v) -- whole groups of v -- and a new definition (get_update(k)), scheduled
      * after it at that level, takes the rest (reference: tiramisu_core.cpp:746-870). */
    void separate(int dim, expr N, int v, expr lower_bound);
    void separate(int dim, expr N, int v) { separate(dim, N, v, expr((int32_t)0)); }
    /** Cut at the given points of loop level \p level: this computation keeps [.., p0), new definitions take
      * [p0, p1), ..., [p(n-1), max) (reference: tiramisu_core.cpp:872-1010). */
    void separate_at(var level, std::vector<expr> separate_points, expr max);
    /** separate() at the loop's own bounds, then split the full part by \p sizeX counting from the loop's lower
      * bound; false when the loop is not longer than sizeX and nothing was split
      * (reference: tiramisu_core.cpp:6103-6240). */
    bool separateAndSplit(var L0, int sizeX);
    bool separateAndSplit(var L0, int sizeX, var L0_outer, var L0_inner);
    bool separateAndSplit(int L0, int sizeX);
    virtual void split_with_lower_bound(int L0, int sizeX, std::string lower_bound);
    /** A copy of this computation (same expression, data mapping and schedule) restricted to the given part of
      * the iteration domain and / or of the time-space domain; scheduled on its own from then on
      * (reference: tiramisu_core.cpp:3244-3310).  select(k) returns the k-th duplicate (0: this computation). */
    computation *duplicate(std::string domain_constraints, std::string range_constraints);
    computation *select(int duplicate_id);
    /** Compute this computation inside the loop nest of \p consumer at loop level \p L: ordered before the
      * consumer there, and whatever the consumer's iterations of that level read that this computation does not
      * produce in the same iteration is computed again by a duplicate, shifted into that iteration
      * (reference: tiramisu_core.cpp:5262-5660). */
    void compute_at(computation &consumer, var L);
    void compute_at(computation &consumer, int L);
    /** Store dimension \p dim of this computation's buffer modulo \p f: the buffer keeps f entries there
      * (reference: tiramisu_core.cpp:8169-8260). */
    virtual void storage_fold(var dim, int f);

    void set_low_level_schedule(std::string map_str);
    void apply_transformation_on_schedule(std::string map_str);
    void set_loop_level_names(std::vector<std::string> names);
    void set_loop_level_names(std::vector<int> loop_levels, std::vector<std::string> names);
    void add_schedule_constraint(std::string domain_constraints, std::string range_constraints);
    int compute_maximal_AST_depth();

    // ---- GPU mapping (reference: tiramisu_core.cpp:358-566, :2498-2580) ----
    virtual void gpu_tile(var L0, var L1, int sizeX, int sizeY);
    virtual void gpu_tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer,
                          var L0_inner, var L1_inner);
    virtual void gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ);
    virtual void gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer,
                          var L1_outer, var L2_outer, var L0_inner, var L1_inner, var L2_inner);
    void tag_gpu_level(var L0, var L1);
    void tag_gpu_level(var L0, var L1, var L2, var L3);
    void tag_gpu_level(var L0, var L1, var L2, var L3, var L4, var L5);
    void tag_gpu_level(int L0, int L1);
    void tag_gpu_level(int L0, int L1, int L2, int L3);
    void tag_gpu_level(int L0, int L1, int L2, int L3, int L4, int L5);
    void tag_gpu_block_level(int L0);
    void tag_gpu_block_level(int L0, int L1);
    void tag_gpu_block_level(int L0, int L1, int L2);
    void tag_gpu_thread_level(int L0);
    void tag_gpu_thread_level(int L0, int L1);
    void tag_gpu_thread_level(int L0, int L1, int L2);
    /** Stage the part of \p inp that one thread block reads in LDS: a cooperative copy
      * at loop level \p level of a tile of \p buffer_shape elements starting at
      * \p copy_offsets, bracketed by barriers (reference: tiramisu_core.cpp:9297-9534). */
    computation *cache_shared(computation &inp, const var &level, const std::vector<int> buffer_shape,
                              const std::vector<expr> copy_offsets, bool pad_buffer = false);
    std::vector<int> thread_block_shape;

    void gen_time_space_domain();
};

class input : public computation {
public:
    input(std::string name, std::vector<var> iterator_variables, primitive_t t);
    input(std::vector<var> iterator_variables, primitive_t t);
    input(std::string name, std::vector<std::string> dimension_names,
          std::vector<expr> dimension_sizes, primitive_t t);
};

/** A named window on a buffer: indexed like a computation, computes nothing and is not scheduled; map it with
  * store_in() to read (or name) what other computations stored there (reference: core.h:5159-5203). */
class view : public computation {
public:
    view(std::string name, std::vector<var> iterator_variables, primitive_t t);
};

class Input : public input {
public:
    Input(std::string name, std::vector<expr> sizes, primitive_t t);
    std::vector<var> iterators_from_size_expressions(std::vector<expr> sizes);
};

class constant : public computation {
public:
    /** Function-wide constant (an invariant): becomes a parameter of every iteration domain
      * declared afterwards and a const scalar at function entry
      * (reference: tiramisu_core.cpp:8178-8283). */
    constant(std::string param_name, const expr &param_expr);
    constant(std::string param_name, const expr &param_expr, primitive_t t, function *func);
    constant(std::string param_name, const expr &param_expr, primitive_t t, bool function_wide,
             computation *with_computation, int at_loop_level, function *func = nullptr /* the implicit function */);
    operator expr();
};

}  // namespace tiramisu
#endif
