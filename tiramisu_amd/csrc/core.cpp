// function / buffer / computation: declaration of iteration domains, the schedule algebra
// and the GPU mapping commands.  Schedules are isl maps from the iteration domain to a
// time-space vector [dup, s0, d0, s1, d1, ..., d(n-1), sn] (static ordering dimensions s_k
// interleaved with dynamic loop dimensions d_k), as in the reference
// (src/tiramisu_core.cpp:2041-2081, :7640-7662); every command is a rewrite of the range.
#include <csignal>
#include <sys/wait.h>
#include <unistd.h>
#include <tiramisu/block.h>
#include <tiramisu/core.h>

#include <algorithm>
#include <cassert>
#include <cstdlib>
#include <queue>
#include <sstream>

#include <tiramisu/isl_api.h>
#include "lir.h"
#include "util.h"

namespace tiramisu {

const var computation::root = var("root");

// ------------------------------------------------------------------ helpers

std::string expr_to_isl_str(const expr &e, bool &ok) {
    if (!e.is_defined()) { ok = false; return ""; }
    switch (e.get_expr_type()) {
    case e_val:
        if (is_float_type(e.get_data_type())) { ok = false; return ""; }
        return std::to_string(e.get_int_val());
    case e_var: return e.get_name();
    case e_op: {
        auto sub = [&](int i) { return expr_to_isl_str(e.get_operand(i), ok); };
        switch (e.get_op_type()) {
        case o_add: return "(" + sub(0) + " + " + sub(1) + ")";
        case o_sub: return "(" + sub(0) + " - " + sub(1) + ")";
        case o_minus: return "(-" + sub(0) + ")";
        case o_mul:
            if (!e.get_operand(0).is_integer_literal() && !e.get_operand(1).is_integer_literal()) ok = false;
            return "(" + sub(0) + " * " + sub(1) + ")";
        case o_div:
            if (!e.get_operand(1).is_integer_literal()) ok = false;
            return "floor(" + sub(0) + " / " + sub(1) + ")";
        case o_mod:
            if (!e.get_operand(1).is_integer_literal()) ok = false;
            return "(" + sub(0) + " mod " + sub(1) + ")";
        case o_max: return "max(" + sub(0) + ", " + sub(1) + ")";
        case o_min: return "min(" + sub(0) + ", " + sub(1) + ")";
        case o_cast:
            if (is_float_type(e.get_data_type())) ok = false;
            return sub(0);
        default: ok = false; return "";
        }
    }
    default: ok = false; return "";
    }
}

static std::string single_piece_text(isl_pw_aff *pa);

static std::string params_prefix(const std::vector<std::string> &params) {
    if (params.empty()) return "";
    return "[" + join(params, ", ") + "] -> ";
}

// ------------------------------------------------------------------ init / codegen

static std::map<std::string, std::string> &command_line_options() {
    static std::map<std::string, std::string> o;
    return o;
}

int backend_options_from_command_line(int argc, char **argv) {
    int taken = 0;
    for (int i = 1; i < argc; i++) {
        std::string a = argv[i], kv;
        if (a == "--backend-option" && i + 1 < argc) kv = argv[++i];
        else if (a.rfind("--backend-option=", 0) == 0) kv = a.substr(17);
        else continue;
        const size_t eq = kv.find('=');
        if (eq == std::string::npos || eq == 0) ERROR("--backend-option wants name=value, got: " + kv, true);
        command_line_options()[kv.substr(0, eq)] = kv.substr(eq + 1);
        taken++;
    }
    return taken;
}

void init(std::string name) {
    function *f = new function(name);
    global::set_implicit_function(f);
    for (auto &o : command_line_options()) f->set_backend_option(o.first, o.second);
}

void init() { init("foo"); }

void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename, const bool gen_gpu) {
    global::get_implicit_function()->codegen(arguments, obj_filename, gen_gpu);
}

void codegen(const std::vector<buffer *> &arguments, const std::string obj_filename,
             const hardware_architecture_t arch) {
    global::get_implicit_function()->codegen(arguments, obj_filename, arch);
}

// ---- options of the back-end.  While a function's code is generated it is the scope of every lookup.
static const function *option_scope = nullptr;
namespace {
struct option_scope_guard {
    const function *saved;
    explicit option_scope_guard(const function *f) : saved(option_scope) { option_scope = f; }
    ~option_scope_guard() { option_scope = saved; }
};
std::string option_name_of(const char *env_name) {
    std::string n = env_name;
    if (n.rfind("TIRAMISU_", 0) == 0) n = n.substr(9);
    for (char &c : n) c = (char)std::tolower((unsigned char)c);
    return n;
}
}  // namespace

void function::set_backend_option(const std::string &name_in, const std::string &value) {
    std::string n = name_in;
    for (char &c : n) c = (char)std::tolower((unsigned char)c);
    if (n.rfind("tiramisu_", 0) == 0) n = n.substr(9);
    if (n.empty()) ERROR("set_backend_option: empty option name", true);
    if (value.empty()) backend_options.erase(n);
    else backend_options[n] = value;
}

const char *function::backend_option(const char *env_name) const {
    const std::string n = option_name_of(env_name);
    const char *v = std::getenv(env_name);
    const char *from = "environment";
    if (!v) {
        auto it = backend_options.find(n);
        if (it == backend_options.end()) return nullptr;
        v = it->second.c_str();
        from = "program";
    }
    for (auto &c : consulted_options)
        if (c[0] == n) return v;
    consulted_options.push_back({n, v, from});
    return v;
}

void set_backend_option(const std::string &name, const std::string &value) {
    if (!global::get_implicit_function()) ERROR("declare a function (tiramisu::init) before setting back-end options", true);
    global::get_implicit_function()->set_backend_option(name, value);
}
void set_backend_option(const std::string &name, long value) { set_backend_option(name, std::to_string(value)); }

const char *backend_option(const char *env_name) {
    const function *f = option_scope ? option_scope : global::get_implicit_function();
    return f ? f->backend_option(env_name) : std::getenv(env_name);
}

static std::map<hardware_architecture_t, backend *> &backend_table() {
    static std::map<hardware_architecture_t, backend *> t;
    return t;
}
void backend::register_backend(hardware_architecture_t arch, backend *b) { backend_table()[arch] = b; }
backend *backend::find(hardware_architecture_t arch) {
    auto it = backend_table().find(arch);
    return it == backend_table().end() ? nullptr : it->second;
}

// ------------------------------------------------------------------ function

function::function(std::string nm) : name(nm) {
    ctx = isl_ctx_alloc();
    if (nm.empty()) ERROR("a function needs a name", true);
}

function::~function() {}

std::vector<computation *> function::get_computation_by_name(std::string nm) const {
    std::vector<computation *> r;
    for (auto c : body)
        if (c->get_name() == nm) r.push_back(c);
    return r;
}

std::vector<std::string> function::get_invariant_names() const {
    std::vector<std::string> r;
    for (auto c : invariants) r.push_back(c->get_name());
    return r;
}

void function::add_computation(computation *c) {
    body.push_back(c);
    if (c->should_schedule_this_computation()) starting_computations.insert(c);
}

void function::add_invariant(constant *c) { invariants.push_back(c); }

void function::add_buffer(std::pair<std::string, buffer *> b) {
    if (buffers_list.count(b.first)) ERROR("buffer " + b.first + " declared twice", true);
    buffers_list[b.first] = b.second;
}

void function::add_context_constraints(std::string s) {
    isl_set *c = isl_set_read_from_str(ctx, s.c_str());
    if (!c) ERROR("cannot parse context " + s, true);
    context_set = context_set ? isl_set_intersect(context_set, c) : c;
}

std::string function::generate_new_name(const std::string &prefix) {
    return prefix + std::to_string(name_counter++);
}

void function::add_parallel_dimension(std::string comp, int level) { parallel_dimensions.insert({comp, level}); }
void function::add_vector_dimension(std::string comp, int level, int length) { vector_dimensions[{comp, level}] = length; }
void function::add_unroll_dimension(std::string comp, int level, int factor) { unroll_dimensions[{comp, level}] = factor; }

void function::add_gpu_block_dimensions(std::string comp, int l0, int l1, int l2) {
    for (auto &p : gpu_block_dimensions)
        if (p.first == comp) { p.second = std::make_tuple(l0, l1, l2); return; }
    gpu_block_dimensions.push_back({comp, std::make_tuple(l0, l1, l2)});
}
void function::add_gpu_thread_dimensions(std::string comp, int l0, int l1, int l2) {
    for (auto &p : gpu_thread_dimensions)
        if (p.first == comp) { p.second = std::make_tuple(l0, l1, l2); return; }
    gpu_thread_dimensions.push_back({comp, std::make_tuple(l0, l1, l2)});
}

bool function::should_parallelize(const std::string &comp, int level) const {
    return parallel_dimensions.count({comp, level}) > 0;
}
int function::vector_length(const std::string &comp, int level) const {
    auto it = vector_dimensions.find({comp, level});
    return it == vector_dimensions.end() ? 0 : it->second;
}
bool function::should_unroll(const std::string &comp, int level) const {
    return unroll_dimensions.count({comp, level}) > 0;
}

// x/y/z are given to the tagged levels from the innermost outwards, so that the
// fastest-varying tagged loop becomes the x index (reference: tiramisu_codegen_cuda.cpp:560-617).
static int position_in(const std::tuple<int, int, int> &t, int level) {
    int lv[3] = {std::get<2>(t), std::get<1>(t), std::get<0>(t)};
    int pos = 0;
    for (int i = 0; i < 3; i++) {
        if (lv[i] == -1) continue;
        if (lv[i] == level) return pos;
        pos++;
    }
    return -1;
}
int function::gpu_block_position(const std::string &comp, int level) const {
    for (auto &p : gpu_block_dimensions)
        if (p.first == comp) return position_in(p.second, level);
    return -1;
}
int function::gpu_thread_position(const std::string &comp, int level) const {
    for (auto &p : gpu_thread_dimensions)
        if (p.first == comp) return position_in(p.second, level);
    return -1;
}

void function::set_arguments(const std::vector<buffer *> &buffer_vec) {
    function_arguments = buffer_vec;
    for (auto b : buffer_vec) {
        if (!b) ERROR("null buffer passed as a function argument", true);
        if (b->location != memory_location::host && b->location != memory_location::global)
            ERROR("argument buffer " + b->get_name() + " must live in host or GPU global memory", true);
    }
}

int function::get_max_schedules_range_dim() const {
    int m = 0;
    for (auto c : body)
        if (c->schedule) m = std::max(m, (int)isl_map_dim(c->schedule, isl_dim_out));
    return m;
}

void function::align_schedules() {
    int m = get_max_schedules_range_dim();
    for (auto c : body) {
        if (!c->schedule) continue;
        int r = isl_map_dim(c->schedule, isl_dim_out);
        if (r == m) continue;
        std::vector<std::string> in, out;
        for (int i = 0; i < r; i++) { in.push_back("x" + std::to_string(i)); out.push_back(in.back()); }
        for (int i = r; i < m; i++) out.push_back("0");
        c->apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    }
}

void function::gen_ordering_schedules() {
    if (use_low_level_scheduling_commands) return;
    // Scheduled computations without a predecessor, in declaration order.
    std::vector<computation *> roots;
    for (auto c : body)
        if (c->should_schedule_this_computation() && starting_computations.count(c)) roots.push_back(c);
    computation *last = nullptr;
    for (auto start : roots) {
        if (last) start->after_low_level(*last, computation::root_dimension);
        // Walk the tree, always descending into the deepest pending fuse level first
        // (reference: tiramisu_function.cpp:2249-2287).
        std::priority_queue<int> level_to_check;
        std::map<int, std::deque<computation *>> level_queue;
        computation *current = start;
        while (true) {
            // deterministic order: successors sorted by declaration order
            std::vector<std::pair<computation *, int>> edges(sched_graph[current].begin(), sched_graph[current].end());
            std::sort(edges.begin(), edges.end(), [&](auto &a, auto &b) {
                return std::find(body.begin(), body.end(), a.first) < std::find(body.begin(), body.end(), b.first);
            });
            for (auto &e : edges) {
                if (level_queue[e.second].empty()) level_to_check.push(e.second);
                level_queue[e.second].push_back(e.first);
            }
            if (level_to_check.empty()) break;
            int fuse_level = level_to_check.top();
            computation *next = level_queue[fuse_level].front();
            level_queue[fuse_level].pop_front();
            next->after_low_level(*current, fuse_level);
            current = next;
            if (level_queue[fuse_level].empty()) level_to_check.pop();
        }
        last = current;
    }
}

void function::gen_time_space_domain() {
    // an update without a mapping of its own stores where its first definition stores
    for (auto c : body)
        if (!c->is_first_definition() && !c->get_access_relation() && c->get_first_definition()->get_access_relation())
            c->set_access(isl_map_copy(c->get_first_definition()->get_access_relation()));
    gen_ordering_schedules();
    align_schedules();
    for (auto c : body) c->gen_time_space_domain();
}

void function::dump_sched_graph() {
    for (auto &a : sched_graph)
        for (auto &b : a.second)
            std::cout << a.first->get_name() << " => " << b.first->get_name() << " [" << b.second << "]\n";
}

void function::dump_schedule() const {
    for (auto c : body) c->dump_schedule();
}

void function::dump(bool) const {
    std::cout << "function " << name << "\n";
    for (auto c : body) c->dump();
}

void function::codegen(const std::vector<buffer *> &arguments, const std::string obj_filename, const bool gen_gpu) {
    codegen(arguments, obj_filename,
            gen_gpu ? hardware_architecture_t::arch_amd_gpu : hardware_architecture_t::arch_cpu);
}

computation *function::get_first_cpt() {
    computation *c = nullptr;
    if (!sched_graph.empty()) c = sched_graph.begin()->first;
    else
        for (auto q : body)
            if (q->should_schedule_this_computation()) { c = q; break; }
    while (c && c->get_predecessor()) c = c->get_predecessor();
    return c;
}

computation *function::get_last_cpt() {
    computation *c = nullptr;
    if (!sched_graph.empty()) c = sched_graph.begin()->first;
    else
        for (auto q : body)
            if (q->should_schedule_this_computation()) { c = q; break; }
    while (c && c->get_successor()) c = c->get_successor();
    return c;
}

void function::Automatic_communication(computation *c1, computation *c2) {
    if (!c1 || !c2) ERROR("automatic CPU/GPU copies need a first and a last computation", true);
    if (c1->get_predecessor()) ERROR("Automatic_communication: " + c1->get_name() + " has a predecessor", true);
    if (c2->get_successor()) ERROR("Automatic_communication: " + c2->get_name() + " has a successor", true);
    computation *first = c1, *last = c2;
    int n = 1;
    for (auto &kv : mapping) {
        buffer *cpu = buffers_list.at(kv.first), *gpu = kv.second;
        if (gpu->get_argument_type() != a_temporary)
            ERROR("buffer " + gpu->get_name() + ": the GPU counterpart of a CPU buffer must be a temporary", true);
        if (!gpu->get_automatic_gpu_copy()) continue;     // the program copies by hand
        const bool to_constant = gpu->get_location() == memory_location::constant;
        if (cpu->get_argument_type() == a_input) {
            computation *c = new computation("cpt" + std::to_string(n++), {}, memcpy(*cpu, *gpu));
            c->then(*first, computation::root);
            first = c;
        }
        if (!to_constant && cpu->get_argument_type() == a_output) {
            computation *c = new computation("cpt" + std::to_string(n++), {}, memcpy(*gpu, *cpu));
            last->then(*c, computation::root);
            last = c;
        }
    }
}

void function::codegen(const std::vector<buffer *> &arguments, const std::string obj_filename_in,
                       hardware_architecture_t arch) {
    option_scope_guard scope(this);
    clear_consulted_backend_options();
    if (arch == hardware_architecture_t::arch_nvidia_gpu) arch = hardware_architecture_t::arch_amd_gpu;
    // mapped buffers get their copies inserted for a GPU target (reference: tiramisu_function.cpp:2542-2549)
    if (arch == hardware_architecture_t::arch_amd_gpu && !mapping.empty())
        Automatic_communication(get_first_cpt(), get_last_cpt());
    std::string obj_filename = obj_filename_in;
    // TIRAMISU_FORCE_ARCH=cpu compiles a GPU program for the host instead (GPU-mapped loops run
    // serially) and writes <name>_cpu.o: how the parity tests obtain CPU-generated code for the
    // very same Tiramisu program.
    if (const char *force = std::getenv("TIRAMISU_FORCE_ARCH")) {
        if (std::string(force) == "cpu" && arch != hardware_architecture_t::arch_cpu) {
            arch = hardware_architecture_t::arch_cpu;
            size_t dot = obj_filename.rfind(".o");
            if (dot != std::string::npos && dot + 2 == obj_filename.size()) obj_filename.insert(dot, "_cpu");
            else obj_filename += "_cpu";
        }
    }
    backend *b = backend::find(arch);
    if (!b) {
        if (arch == hardware_architecture_t::arch_cpu)
            ERROR("no CPU back-end is linked into this program: the GPU library generates HIP only; "
                  "link the oracle's CPU emitter to generate host code", true);
        ERROR("no back-end registered for the requested architecture", true);
    }
    set_arguments(arguments);
    gen_time_space_domain();
    if (arch == hardware_architecture_t::arch_amd_gpu && backend_option("TIRAMISU_HIP_CHECK_MAPPED_LOOPS")) {
        // The analysis is one isl dataflow computation over the whole function and has no natural bound (a tensor
        // contraction with hundreds of statements: more than 40 minutes), so it runs in a child process with a time
        // limit (option hip_check_time_limit, seconds, default 600; 0: in this process, without one).  A check that
        // does not finish says so and stops nothing.
        const char *limit_text = backend_option("TIRAMISU_HIP_CHECK_TIME_LIMIT");
        const int limit = limit_text ? std::atoi(limit_text) : 600;
        std::vector<std::string> races;
        bool finished = true;
        if (limit <= 0) {
            races = gpu_mapped_loops_that_carry_dependences();
        } else {
            int fd[2];
            if (pipe(fd) != 0) ERROR("pipe() failed", true);
            std::cout.flush();
            std::cerr.flush();
            const pid_t child = fork();
            if (child < 0) ERROR("fork() failed", true);
            if (child == 0) {
                close(fd[0]);
                alarm((unsigned)limit);
                std::string all;
                for (auto &r : gpu_mapped_loops_that_carry_dependences()) all += r + "\n";
                size_t off = 0;
                while (off < all.size()) {
                    const ssize_t n = write(fd[1], all.data() + off, all.size() - off);
                    if (n <= 0) break;
                    off += (size_t)n;
                }
                _exit(0);
            }
            close(fd[1]);
            std::string all;
            char buf[4096];
            for (ssize_t n; (n = read(fd[0], buf, sizeof buf)) > 0;) all.append(buf, (size_t)n);
            close(fd[0]);
            int status = 0;
            waitpid(child, &status, 0);
            finished = WIFEXITED(status) && WEXITSTATUS(status) == 0;
            if (!finished && !(WIFSIGNALED(status) && WTERMSIG(status) == SIGALRM)) ERROR("the check of the GPU mapping ended abnormally", true);
            for (size_t a = 0, b; (b = all.find('\n', a)) != std::string::npos; a = b + 1) races.push_back(all.substr(a, b - a));
        }
        if (!finished)
            std::cerr << "GPU mapping: the dependence analysis of " << name << " did not finish within " << limit
                      << " s and was stopped: its mapped loops are not checked (hip_check_time_limit sets the limit)" << std::endl;
        bool refuse = false;
        for (auto &r : races) {
            std::cerr << "GPU mapping: " << r << std::endl;
            refuse |= r.find("carries a dependence") != std::string::npos;      // a reduction is only reported
        }
        if (refuse) ERROR("loops mapped to the GPU carry dependences", true);
    }
    gen_isl_ast();
    b->generate(*this, get_lowered_program(), obj_filename);
}

void function::gen_halide_obj(const std::string &obj_file_name) {
    option_scope_guard scope(this);
    hardware_architecture_t arch =
        hand_driven_gpu ? hardware_architecture_t::arch_amd_gpu : hardware_architecture_t::arch_cpu;
    // GPU-mapped loops without gen_cuda_stmt(): the reference leaves them to Halide's GPU target
    // (tests/test_17.cpp - test_19.cpp); here they go to the HIP back-end with implicit copies,
    // unless a CPU back-end is linked in and asked for
    if (!hand_driven_gpu && !gpu_block_dimensions.empty() && backend::find(hardware_architecture_t::arch_amd_gpu) &&
        !(std::getenv("TIRAMISU_FORCE_ARCH") && std::string(std::getenv("TIRAMISU_FORCE_ARCH")) == "cpu")) {
        arch = hardware_architecture_t::arch_amd_gpu;
        implicit_gpu_copies = true;
    }
    backend *b = backend::find(arch);
    if (!b) ERROR("no back-end registered for the requested architecture", true);
    if (!ast) gen_isl_ast();
    b->generate(*this, get_lowered_program(), obj_file_name);
}

lir::program &function::get_lowered_program() {
    if (!lowered) ERROR("gen_isl_ast() has not been run", true);
    return *lowered;
}

// ------------------------------------------------------------------ buffer

buffer::buffer(std::string nm, std::vector<expr> sizes, primitive_t t, argument_t argt, function *f,
               std::string corr)
    : name(nm), dim_sizes(std::move(sizes)), type(t), argtype(argt), fct(f) {
    if (!fct) ERROR("declare a function (tiramisu::init) before declaring buffers", true);
    if (name.empty()) ERROR("a buffer needs a name", true);
    for (auto &e : dim_sizes)
        if (!e.is_defined()) ERROR("undefined size expression for buffer " + name, true);
    fct->add_buffer({name, this});
    if (!corr.empty()) {
        // this is the GPU counterpart of CPU buffer `corr` (reference: tiramisu_core.cpp:6775-6779)
        if (!fct->get_buffers().count(corr)) ERROR("buffer " + name + ": no CPU buffer named " + corr, true);
        fct->add_mapping({corr, this});
    }
}

bool buffer::has_constant_extents() const {
    for (auto &e : dim_sizes)
        if (!lir::simplify(e).is_integer_literal()) return false;
    return true;
}

void buffer::tag_gpu_register() {
    bool one = dim_sizes.size() == 1 && lir::simplify(dim_sizes[0]).is_integer_literal() &&
               lir::simplify(dim_sizes[0]).get_int_val() == 1;
    if (!one) ERROR("a register buffer must have the shape {1}: " + name, true);
    location = memory_location::reg;
    auto_allocate = false;
}

void buffer::dump(bool) const {
    std::cout << "buffer " << name << " [";
    for (size_t i = 0; i < dim_sizes.size(); i++) std::cout << (i ? ", " : "") << dim_sizes[i].to_str();
    std::cout << "] " << str_from_tiramisu_type_primitive(type) << "\n";
}

// Allocation / release computations live on the first level+1 dimensions of C's iteration
// domain; the program orders them itself with then()/after()
// (reference: tiramisu_core.cpp:1479-1631).
static computation *make_alloc_like(buffer *b, computation &C, int level, bool is_alloc, function *fct) {
    isl_set *dom = isl_set_copy(C.get_iteration_domain());
    int n = isl_set_dim(dom, isl_dim_set);
    if (level + 1 > n) ERROR("allocate_at/deallocate_at: level out of range", true);
    if (level + 1 == 0) {
        isl_set_free(dom);
        dom = isl_set_read_from_str(C.get_ctx(), "{ [0] }");
    } else {
        dom = isl_set_project_out(dom, isl_dim_set, level + 1, n - (level + 1));
    }
    std::string nm = std::string(is_alloc ? "_allocation_" : "_deallocation_") + C.get_name();
    dom = isl_set_set_tuple_name(dom, nm.c_str());
    char *s = isl_set_to_str(dom);
    std::string dom_str(s);
    free(s);
    isl_set_free(dom);
    expr e = is_alloc ? expr(o_allocate, b->get_name()) : expr(o_free, b->get_name());
    computation *a = new computation(dom_str, e, true, p_none, fct);
    std::vector<std::string> names(C.get_loop_level_names().begin(), C.get_loop_level_names().begin() + level + 1);
    a->set_loop_level_names(names);
    return a;
}

computation *buffer::allocate_at(computation &C, int level) {
    set_auto_allocate(false);
    return make_alloc_like(this, C, level, true, fct);
}
computation *buffer::allocate_at(computation &C, var level) {
    return allocate_at(C, C.get_loop_level_number_from_dimension_name(level.get_name()));
}
computation *buffer::deallocate_at(computation &C, int level) {
    set_auto_deallocate(false);
    return make_alloc_like(this, C, level, false, fct);
}
computation *buffer::deallocate_at(computation &C, var level) {
    return deallocate_at(C, C.get_loop_level_number_from_dimension_name(level.get_name()));
}

// ------------------------------------------------------------------ computation: construction

computation::~computation() {}

std::string computation::construct_iteration_domain(const std::string &nm, const std::vector<var> &vars) {
    std::vector<std::string> params = fct->get_invariant_names();
    std::ostringstream os;
    os << params_prefix(params) << "{ " << nm << "[";
    if (vars.empty()) {
        os << "0] }";
        return os.str();
    }
    for (size_t i = 0; i < vars.size(); i++) os << (i ? ", " : "") << vars[i].get_name();
    os << "] : ";
    for (size_t i = 0; i < vars.size(); i++) {
        bool ok = true;
        if (!vars[i].get_lower().is_defined() || !vars[i].get_upper().is_defined())
            ERROR("iterator " + vars[i].get_name() + " of " + nm + " has no bounds", true);
        std::string lo = expr_to_isl_str(vars[i].get_lower(), ok);
        std::string up = expr_to_isl_str(vars[i].get_upper(), ok);
        if (!ok) ERROR("bounds of iterator " + vars[i].get_name() + " are not affine", true);
        os << (i ? " and " : "") << lo << " <= " << vars[i].get_name() << " < " << up;
    }
    os << " }";
    return os.str();
}

void computation::init_computation(std::string iteration_space_str, function *f, const expr &e,
                                   bool schedule_this_computation, primitive_t t) {
    fct = f;
    if (!fct) ERROR("declare a function (tiramisu::init) before declaring computations", true);
    ctx = fct->get_isl_ctx();
    iteration_domain = isl_set_read_from_str(ctx, iteration_space_str.c_str());
    if (!iteration_domain) ERROR("cannot parse iteration domain: " + iteration_space_str, true);
    const char *tn = isl_set_get_tuple_name(iteration_domain);
    if (!tn) ERROR("iteration domain without a name: " + iteration_space_str, true);
    name = tn;
    int n = isl_set_dim(iteration_domain, isl_dim_set);
    iterator_names_.clear();
    for (int i = 0; i < n; i++) {
        const char *dn = isl_set_get_dim_name(iteration_domain, isl_dim_set, i);
        iterator_names_.push_back(dn ? dn : ("_i" + std::to_string(i)));
    }
    level_names = iterator_names_;
    expression = e;
    data_type = t;
    schedule_this = schedule_this_computation;
    set_identity_schedule();
    fct->add_computation(this);
}

void computation::set_identity_schedule() {
    int n = (int)iterator_names_.size();
    std::vector<std::string> in, out{"0", "0"};
    for (int i = 0; i < n; i++) {
        in.push_back("t" + std::to_string(i));
        out.push_back(in.back());
        out.push_back("0");
    }
    std::string s = "{ " + name + "[" + join(in, ",") + "] -> [" + join(out, ",") + "] }";
    schedule = isl_map_read_from_str(ctx, s.c_str());
}

computation::computation(std::string iteration_domain_str, expr e, bool schedule_this_computation,
                         primitive_t t, function *f) {
    init_computation(iteration_domain_str, f, e, schedule_this_computation, t);
}

computation::computation(std::string nm, std::vector<var> iterator_variables, expr e,
                         bool schedule_this_computation) {
    fct = global::get_implicit_function();
    if (!fct) ERROR("call tiramisu::init() first", true);
    declared_vars = iterator_variables;
    init_computation(construct_iteration_domain(nm, iterator_variables), fct, e, schedule_this_computation,
                     e.get_data_type());
    if (iterator_variables.empty()) { iterator_names_ = {"_zero"}; level_names = iterator_names_; }
    if (global::is_auto_data_mapping_set() && has_accesses()) allocate_and_map_buffer_automatically(a_temporary);
}

static std::string fresh_computation_name() {
    static int n = 0;
    return "_comp" + std::to_string(n++);
}

computation::computation(std::vector<var> iterator_variables, expr e)
    : computation(fresh_computation_name(), iterator_variables, e, true) {}
computation::computation(std::string nm, std::vector<var> iterator_variables, expr e)
    : computation(nm, iterator_variables, e, true) {}
computation::computation(std::vector<var> iterator_variables, expr p, expr e)
    : computation(fresh_computation_name(), iterator_variables, e, true) { add_predicate(p); }
computation::computation(std::string nm, std::vector<var> iterator_variables, expr p, expr e)
    : computation(nm, iterator_variables, e, true) { add_predicate(p); }
computation::computation(std::vector<var> iterator_variables, expr e, bool schedule_this_computation)
    : computation(fresh_computation_name(), iterator_variables, e, schedule_this_computation) {}

bool computation::has_accesses() const {
    // Leaves that only act (barrier, copy, allocation, library call) store nothing
    // (reference: tiramisu_core.cpp:7797-7813).
    if (expression.get_expr_type() == e_sync) return false;
    if (expression.get_expr_type() == e_op) {
        op_t o = expression.get_op_type();
        if (o == o_memcpy || o == o_allocate || o == o_free) return false;
    }
    if (is_let) return false;
    return true;
}

int computation::get_iteration_domain_dimensions_number() const {
    return isl_set_dim(iteration_domain, isl_dim_set);
}

void computation::allocate_and_map_buffer_automatically(argument_t type) {
    std::vector<expr> sizes;
    const int ndims = isl_set_dim(iteration_domain, isl_dim_set);
    if (declared_vars.empty() && ndims > 0 && iterator_names_ != std::vector<std::string>{"_zero"}) {
        // domain given as an isl string: one buffer dimension per iterator, largest value + 1
        for (int d = 0; d < ndims; d++) sizes.push_back(lir::extent_of_dimension(fct, iteration_domain, d));
    } else if (declared_vars.empty()) {
        sizes.push_back(expr((int32_t)1));
    } else {
        for (auto &v : declared_vars) {
            if (!v.get_upper().is_defined()) return;  // unbounded: the user maps it by hand
            sizes.push_back(lir::simplify(v.get_upper() - v.get_lower()));
        }
    }
    std::string bname = "_" + name + "_" + fct->generate_new_name("b");
    automatically_allocated_buffer = new buffer(bname, sizes, data_type, type, fct);
    store_in(automatically_allocated_buffer);
}

static void collect_reads(const expr &e, std::set<std::string> &names) {
    if (!e.is_defined()) return;
    if (e.get_expr_type() == e_op && e.get_op_type() == o_access) names.insert(e.get_name());
    for (auto &o : e.get_operands()) collect_reads(o, names);
    for (auto &a : e.get_arguments()) collect_reads(a, names);
}

void function::allocate_and_map_buffers_automatically() {
    std::set<std::string> read;
    for (computation *c : body) {
        collect_reads(c->get_expr(), read);
        collect_reads(c->get_predicate(), read);
    }
    for (computation *c : body) {
        if (!c->has_accesses() || c->get_access_relation() || c->get_automatically_allocated_buffer()) continue;
        if (c->is_inline_computation()) continue;    // replaced by its expression wherever it is read: no storage (its domain may be unbounded)
        if (!c->is_first_definition()) continue;      // updates share the first definition's buffer, below
        const argument_t kind = !c->should_schedule_this_computation() ? a_input : (read.count(c->get_name()) ? a_temporary : a_output);
        c->allocate_and_map_buffer_automatically(kind);
    }
    for (computation *c : body)
        if (!c->is_first_definition() && c->has_accesses() && !c->get_access_relation() && c->get_first_definition()->get_buffer())
            c->store_in(c->get_first_definition()->get_buffer());
}

void function::dump_dep_graph() { dump_sched_graph(); }

void function::dump_iteration_domain() const {
    for (auto c : body) c->dump_iteration_domain();
}

void function::dump_time_processor_domain() const {
    for (auto c : body) {
        isl_set *ts = isl_set_apply(isl_set_copy(c->get_iteration_domain()), isl_map_copy(c->get_schedule()));
        char *str = isl_set_to_str(ts);
        std::cout << c->get_name() << ": " << str << std::endl;
        free(str);
        isl_set_free(ts);
    }
}

constant *function::get_invariant_by_name(std::string str) const {
    for (auto c : invariants)
        if (c->get_name() == str) return static_cast<constant *>(c);
    return nullptr;
}

buffer *computation::get_buffer() const {
    if (!access) return nullptr;
    const char *bn = isl_map_get_tuple_name(access, isl_dim_out);
    if (!bn) return nullptr;
    auto it = fct->get_buffers().find(bn);
    return it == fct->get_buffers().end() ? nullptr : it->second;
}

void computation::set_expression(const expr &e) {
    expression = e;
    if (data_type == p_none) data_type = e.get_data_type();
}

void computation::set_access(std::string access_str) {
    isl_map *m = isl_map_read_from_str(ctx, access_str.c_str());
    if (!m) ERROR("cannot parse access relation " + access_str, true);
    set_access(m);
}

void computation::set_access(isl_map *acc) {
    if (access) isl_map_free(access);
    // an update is addressed by the name of its first definition in the relations the user writes
    if (first_definition && acc) acc = isl_map_set_tuple_name(acc, isl_dim_in, name.c_str());
    access = acc;
}

void computation::add_definitions(std::string iteration_domain_str, expr e, bool schedule_this_computation, primitive_t t, function *f) {
    if (first_definition) ERROR("add_definitions: call it on the first definition of " + first_definition->get_name(), true);
    isl_set *dom = isl_set_read_from_str(ctx, iteration_domain_str.c_str());
    if (!dom) ERROR("cannot parse iteration domain " + iteration_domain_str, true);
    const std::string update_name = "_" + name + "_update_" + std::to_string(updates.size() + 1);
    dom = isl_set_set_tuple_name(dom, update_name.c_str());
    char *text = isl_set_to_str(dom);
    computation *c = new computation(std::string(text), e, schedule_this_computation, t, f);
    free(text);
    isl_set_free(dom);
    c->first_definition = this;
    c->is_let = is_let;
    updates.push_back(c);
}

computation *computation::store_at(computation &comp, var L0) {
    const int level = comp.get_loop_level_number_from_dimension_name(L0.get_name());
    allocate_and_map_buffer_automatically(a_temporary);
    if (!automatically_allocated_buffer) ERROR("store_at: the size of " + name + " is not known", true);
    computation *allocation = automatically_allocated_buffer->allocate_at(comp, level);
    if (comp.get_predecessor()) allocation->between(*comp.get_predecessor(), L0, comp, L0);
    else allocation->before(comp, level);
    return allocation;
}

computation &computation::get_update(int index) {
    if (index == 0) return *this;
    if (index < 0 || index > (int)updates.size()) ERROR("get_update: " + name + " has no definition number " + std::to_string(index), true);
    return *updates[index - 1];
}

void computation::store_in(buffer *buff) {
    std::vector<expr> idx;
    int n = (int)iterator_names_.size();
    // A buffer with fewer dimensions than the domain takes the innermost iterators.
    int nb = buff->get_n_dims();
    for (int i = std::max(0, n - nb); i < n; i++) idx.push_back(var(iterator_names_[i]));
    if (iterator_names_ == std::vector<std::string>{"_zero"}) idx = {expr((int32_t)0)};   // a computation without iterators
    store_in(buff, idx);
}

void computation::store_in(buffer *buff, std::vector<expr> iterators) {
    // no index at all: every iteration stores into element 0 (a scalar kept in a one-element buffer)
    if (iterators.empty()) iterators.assign(std::max(1, buff->get_n_dims()), expr((int32_t)0));
    std::vector<std::string> out;
    for (auto &e : iterators) {
        bool ok = true;
        out.push_back(expr_to_isl_str(e, ok));
        if (!ok) ERROR("store_in of " + name + ": index " + e.to_str() + " is not affine", true);
    }
    const std::vector<std::string> &in = iterator_names_;
    std::string s = params_prefix(fct->get_invariant_names()) + "{ " + name + "[" + join(in, ", ") + "] -> " +
                    buff->get_name() + "[" + join(out, ", ") + "] }";
    set_access(s);
}

void computation::store_in(std::vector<expr> mapping, std::vector<expr> sizes) {
    std::string bname = "_" + name + "_" + fct->generate_new_name("b");
    buffer *b = new buffer(bname, sizes, data_type, a_temporary, fct);
    automatically_allocated_buffer = b;
    store_in(b, mapping);
}

expr computation::make_access(const std::vector<expr> &idx) {
    if ((int)idx.size() != (int)iterator_names_.size() && !(declared_vars.empty() && idx.empty())) {
        std::string s = "Error - Incorrect access: " + name + "(";
        for (size_t i = 0; i < idx.size(); i++) s += (i ? ", " : "") + idx[i].to_str();
        ERROR(s + "). The number of access dimensions does not match the declaration of " + name, true);
    }
    if (inline_) {
        std::map<std::string, expr> subs;
        for (size_t i = 0; i < idx.size(); i++) subs[iterator_names_[i]] = idx[i];
        return expression.substitute(subs);
    }
    return expr(o_access, name, idx, data_type);
}

computation::operator expr() {
    std::vector<expr> idx;
    for (auto &n : iterator_names_) idx.push_back(var(n));
    return make_access(idx);
}

void computation::dump_iteration_domain() const {
    char *s = isl_set_to_str(iteration_domain);
    std::cout << s << std::endl;
    free(s);
}
void computation::dump_schedule() const {
    char *s = isl_map_to_str(schedule);
    std::cout << name << ": " << s << "   levels: " << join(level_names, ",") << std::endl;
    free(s);
}
void computation::dump() const {
    dump_iteration_domain();
    dump_schedule();
    std::cout << "  expr: " << expression.to_str() << std::endl;
    if (access) {
        char *s = isl_map_to_str(access);
        std::cout << "  access: " << s << std::endl;
        free(s);
    }
}

// ------------------------------------------------------------------ computation: names and levels

std::vector<int> computation::get_loop_level_numbers_from_dimension_names(const std::vector<std::string> &names) const {
    std::vector<int> r;
    for (auto &n : names) {
        if (n == "root") { r.push_back(root_dimension); continue; }
        auto it = std::find(level_names.begin(), level_names.end(), n);
        if (it == level_names.end())
            ERROR("dimension " + n + " not found in the schedule of " + name + " (levels: " + join(level_names, ",") + ")", true);
        r.push_back((int)(it - level_names.begin()));
    }
    return r;
}

void computation::set_loop_level_names(std::vector<std::string> names) {
    for (size_t i = 0; i < names.size() && i < level_names.size(); i++) level_names[i] = names[i];
}
void computation::set_loop_level_names(std::vector<int> loop_levels, std::vector<std::string> names) {
    for (size_t i = 0; i < loop_levels.size(); i++) level_names.at(loop_levels[i]) = names[i];
}

void computation::assert_names_not_assigned(const std::vector<std::string> &names) const {
    for (auto &n : names)
        if (std::find(level_names.begin(), level_names.end(), n) != level_names.end())
            ERROR("dimension name " + n + " is already used in the schedule of " + name, true);
}

void computation::apply_on_range(const std::string &t) {
    isl_map *m = isl_map_read_from_str(ctx, t.c_str());
    if (!m) ERROR("cannot parse schedule transformation " + t, true);
    // dimensions that align_schedules() appended (zeros behind the last level) are dropped again first
    const int have = (int)isl_map_dim(schedule, isl_dim_out), takes = (int)isl_map_dim(m, isl_dim_in);
    if (have > takes) schedule = isl_map_project_out(schedule, isl_dim_out, takes, have - takes);
    schedule = isl_map_apply_range(schedule, m);
}

void computation::apply_transformation_on_schedule(std::string map_str) { apply_on_range(map_str); }

void computation::set_low_level_schedule(std::string map_str) {
    isl_map *m = isl_map_read_from_str(ctx, map_str.c_str());
    if (!m) ERROR("cannot parse schedule " + map_str, true);
    if (schedule) isl_map_free(schedule);
    schedule = m;
    fct->use_low_level_scheduling_commands = true;
}

void computation::add_schedule_constraint(std::string domain_constraints, std::string range_constraints) {
    if (!domain_constraints.empty()) {
        isl_set *d = isl_set_read_from_str(ctx, domain_constraints.c_str());
        schedule = isl_map_intersect_domain(schedule, d);
    }
    if (!range_constraints.empty()) {
        isl_set *r = isl_set_read_from_str(ctx, range_constraints.c_str());
        schedule = isl_map_intersect_range(schedule, r);
    }
}

// Range variable lists for a transformation of a schedule with n levels.
static void range_vars(int n, std::vector<std::string> &v) {
    v.clear();
    for (int i = 0; i < 2 * n + 2; i++) v.push_back("x" + std::to_string(i));
}

// ------------------------------------------------------------------ loop transformations

void computation::split(int L0, int sizeX) {
    int n = (int)level_names.size();
    if (L0 < 0 || L0 >= n) ERROR("split: level out of range for " + name, true);
    if (sizeX < 1) ERROR("split: factor must be positive", true);
    std::vector<std::string> in, out;
    range_vars(n, in);
    int p = dynamic_pos(L0);
    for (int i = 0; i < (int)in.size(); i++) {
        if (i == p) { out.push_back("o"); out.push_back("0"); out.push_back("r"); }
        else out.push_back(in[i]);
    }
    std::string s = std::to_string(sizeX);
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] : o = floor(" + in[p] + "/" + s +
                   ") and r = " + in[p] + " - " + s + "*o }");
    std::string base = level_names[L0];
    level_names[L0] = base + "_outer";
    level_names.insert(level_names.begin() + L0 + 1, base + "_inner");
}

void computation::split(var L0, int sizeX, var L0_outer, var L0_inner) {
    int l = get_loop_level_number_from_dimension_name(L0.get_name());
    assert_names_not_assigned({L0_outer.get_name(), L0_inner.get_name()});
    split(l, sizeX);
    level_names[l] = L0_outer.get_name();
    level_names[l + 1] = L0_inner.get_name();
}

void computation::split(var L0, int sizeX) {
    split(L0, sizeX, var(fct->generate_new_name(L0.get_name() + "_o")), var(fct->generate_new_name(L0.get_name() + "_i")));
}

void computation::interchange(int L0, int L1) {
    int n = (int)level_names.size();
    if (L0 < 0 || L1 < 0 || L0 >= n || L1 >= n) ERROR("interchange: level out of range for " + name, true);
    std::vector<std::string> in, out;
    range_vars(n, in);
    out = in;
    std::swap(out[dynamic_pos(L0)], out[dynamic_pos(L1)]);
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    std::swap(level_names[L0], level_names[L1]);
}

void computation::interchange(var L0, var L1) {
    auto l = get_loop_level_numbers_from_dimension_names({L0.get_name(), L1.get_name()});
    interchange(l[0], l[1]);
}

// tile = split both loops, then move the first inner loop below the second outer loop
// (reference: tiramisu_core.cpp:2705-2723).
void computation::tile(int L0, int L1, int sizeX, int sizeY) {
    if (L1 != L0 + 1) ERROR("tile: the two levels must be consecutive", true);
    split(L0, sizeX);
    split(L1 + 1, sizeY);
    interchange(L0 + 1, L1 + 1);
}

void computation::tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer, var L0_inner,
                       var L1_inner) {
    auto l = get_loop_level_numbers_from_dimension_names({L0.get_name(), L1.get_name()});
    assert_names_not_assigned({L0_outer.get_name(), L1_outer.get_name(), L0_inner.get_name(), L1_inner.get_name()});
    tile(l[0], l[1], sizeX, sizeY);
    level_names[l[0]] = L0_outer.get_name();
    level_names[l[0] + 1] = L1_outer.get_name();
    level_names[l[0] + 2] = L0_inner.get_name();
    level_names[l[0] + 3] = L1_inner.get_name();
}

void computation::tile(var L0, var L1, int sizeX, int sizeY) {
    tile(L0, L1, sizeX, sizeY, var(fct->generate_new_name(L0.get_name() + "_o")),
         var(fct->generate_new_name(L1.get_name() + "_o")), var(fct->generate_new_name(L0.get_name() + "_i")),
         var(fct->generate_new_name(L1.get_name() + "_i")));
}

// 3-D tile: order becomes L0o, L1o, L2o, L0i, L1i, L2i (reference: tiramisu_core.cpp:2971-3062).
void computation::tile(int L0, int L1, int L2, int sizeX, int sizeY, int sizeZ) {
    if (L1 != L0 + 1 || L2 != L1 + 1) ERROR("tile: the three levels must be consecutive", true);
    split(L0, sizeX);       // L0o L0i L1 L2
    split(L0 + 2, sizeY);   // L0o L0i L1o L1i L2
    split(L0 + 4, sizeZ);   // L0o L0i L1o L1i L2o L2i
    interchange(L0 + 1, L0 + 2);  // L0o L1o L0i L1i L2o L2i
    interchange(L0 + 2, L0 + 4);  // L0o L1o L2o L1i L0i L2i
    interchange(L0 + 3, L0 + 4);  // L0o L1o L2o L0i L1i L2i
}

void computation::tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer, var L1_outer,
                       var L2_outer, var L0_inner, var L1_inner, var L2_inner) {
    auto l = get_loop_level_numbers_from_dimension_names({L0.get_name(), L1.get_name(), L2.get_name()});
    tile(l[0], l[1], l[2], sizeX, sizeY, sizeZ);
    std::string nm[6] = {L0_outer.get_name(), L1_outer.get_name(), L2_outer.get_name(),
                         L0_inner.get_name(), L1_inner.get_name(), L2_inner.get_name()};
    for (int i = 0; i < 6; i++) level_names[l[0] + i] = nm[i];
}

void computation::tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ) {
    auto g = [&](const var &v, const char *s) { return var(fct->generate_new_name(v.get_name() + s)); };
    tile(L0, L1, L2, sizeX, sizeY, sizeZ, g(L0, "_o"), g(L1, "_o"), g(L2, "_o"), g(L0, "_i"), g(L1, "_i"), g(L2, "_i"));
}

void computation::shift(int L0, int n) {
    std::vector<std::string> in, out;
    range_vars((int)level_names.size(), in);
    out = in;
    out[dynamic_pos(L0)] = in[dynamic_pos(L0)] + " + " + std::to_string(n);
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
}
void computation::shift(var L0, int n) { shift(get_loop_level_number_from_dimension_name(L0.get_name()), n); }

// skew(i, j, f): j' = f*i + j (reference: core.h "skew" documentation).
void computation::skew(int i, int j, int factor) {
    std::vector<std::string> in, out;
    range_vars((int)level_names.size(), in);
    out = in;
    out[dynamic_pos(j)] = std::to_string(factor) + "*" + in[dynamic_pos(i)] + " + " + in[dynamic_pos(j)];
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
}
void computation::skew(var i, var j, int factor) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name()});
    skew(l[0], l[1], factor);
}
void computation::skew(var i, var j, int factor, var ni, var nj) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name()});
    skew(l[0], l[1], factor);
    level_names[l[0]] = ni.get_name();
    level_names[l[1]] = nj.get_name();
}

void computation::skew(int i, int j, int alpha, int beta, int gamma, int sigma) {
    if (i + 1 != j) ERROR("skew: the two loop levels must be consecutive, outer first", true);
    if (std::abs(alpha * sigma - beta * gamma) != 1) ERROR("skew: alpha * sigma - beta * gamma must be 1 or -1", true);
    std::vector<std::string> in, out;
    range_vars((int)level_names.size(), in);
    out = in;
    const std::string &vi = in[dynamic_pos(i)], &vj = in[dynamic_pos(j)];
    out[dynamic_pos(i)] = std::to_string(alpha) + "*" + vi + " + " + std::to_string(beta) + "*" + vj;
    out[dynamic_pos(j)] = std::to_string(gamma) + "*" + vi + " + " + std::to_string(sigma) + "*" + vj;
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
}
bool skewing_second_row(int &a, int &b, int &gamma, int &sigma) {
    // the second row of the unimodular matrix, chosen as the reference chooses it (tiramisu_core.cpp:4445-4497)
    if (b == 0 || a < 0) return false;
    int n1 = std::abs(a), n2 = std::abs(b);
    if (n1 == 0) n1 = n2;
    while (n1 != n2) { if (n1 > n2) n1 -= n2; else n2 -= n1; }
    a /= n1;
    b /= n1;
    gamma = 0;
    sigma = 1;
    if (b == 1 || a == 1) gamma = a - 1;
    else if (b == -1 && a > 1) { gamma = 1; sigma = 0; }
    else {
        bool found = false;
        for (int t = 0; t < 100 && !found; t++) {
            if ((sigma * a) % std::abs(b) == 1) found = true;
            else sigma++;
        }
        if (!found) return false;
        gamma = (sigma * a - 1) / b;
    }
    return true;
}

void computation::skew(int i, int j, int a, int b) {
    int gamma, sigma;
    if (b == 0 || a < 0) ERROR("skew: needs a >= 0 and b != 0", true);
    if (!skewing_second_row(a, b, gamma, sigma)) ERROR("skew: no integer solution of a * sigma - b * gamma = 1", true);
    skew(i, j, a, b, gamma, sigma);
}
void computation::skew(var i, var j, int a, int b, var ni, var nj) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name()});
    skew(l[0], l[1], a, b);
    level_names[l[0]] = ni.get_name();
    level_names[l[1]] = nj.get_name();
}
void computation::skew(var i, var j, int alpha, int beta, int gamma, int sigma, var ni, var nj) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name()});
    skew(l[0], l[1], alpha, beta, gamma, sigma);
    level_names[l[0]] = ni.get_name();
    level_names[l[1]] = nj.get_name();
}
void computation::skew(int i, int j, int k, int l, int factor) {
    skew(i, j, factor);
    skew(i, k, factor);
    skew(i, l, factor);
}
void computation::skew(var i, var j, var k, int factor) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name(), k.get_name()});
    skew(l[0], l[1], factor);
    skew(l[0], l[2], factor);
}
void computation::skew(var i, var j, var k, var l4, int factor) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name(), k.get_name(), l4.get_name()});
    skew(l[0], l[1], l[2], l[3], factor);
}
void computation::skew(var i, var j, var k, int factor, var ni, var nj, var nk) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name(), k.get_name()});
    skew(l[0], l[1], factor);
    skew(l[0], l[2], factor);
    level_names[l[0]] = ni.get_name();
    level_names[l[1]] = nj.get_name();
    level_names[l[2]] = nk.get_name();
}
void computation::skew(var i, var j, var k, var l4, int factor, var ni, var nj, var nk, var nl) {
    auto l = get_loop_level_numbers_from_dimension_names({i.get_name(), j.get_name(), k.get_name(), l4.get_name()});
    skew(l[0], l[1], l[2], l[3], factor);
    level_names[l[0]] = ni.get_name();
    level_names[l[1]] = nj.get_name();
    level_names[l[2]] = nk.get_name();
    level_names[l[3]] = nl.get_name();
}

void computation::loop_reversal(int i) {
    std::vector<std::string> in, out;
    range_vars((int)level_names.size(), in);
    out = in;
    out[dynamic_pos(i)] = "-" + in[dynamic_pos(i)];
    apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
}
void computation::loop_reversal(var old_var, var new_var) {
    int l = get_loop_level_number_from_dimension_name(old_var.get_name());
    loop_reversal(l);
    level_names[l] = new_var.get_name();
}

void computation::tag_parallel_level(int L) { fct->add_parallel_dimension(name, L); }
void computation::tag_parallel_level(var L) { tag_parallel_level(get_loop_level_number_from_dimension_name(L.get_name())); }
void computation::parallelize(var L) { tag_parallel_level(L); }
void computation::tag_vector_level(int L, int len) { fct->add_vector_dimension(name, L, len); }
void computation::tag_vector_level(var L, int len) { tag_vector_level(get_loop_level_number_from_dimension_name(L.get_name()), len); }
void computation::tag_unroll_level(int L) { fct->add_unroll_dimension(name, L, 0); }
void computation::tag_unroll_level(int L, int F) { fct->add_unroll_dimension(name, L, F); }
void computation::tag_unroll_level(var L) { tag_unroll_level(get_loop_level_number_from_dimension_name(L.get_name())); }
void computation::tag_unroll_level(var L, int F) { tag_unroll_level(get_loop_level_number_from_dimension_name(L.get_name()), F); }

// vectorize/unroll: split by the factor and tag the inner loop.  The reference first
// separates a remainder computation when the extent is not a multiple of the factor
// (tiramisu_core.cpp:1238-1370); here the inner loop simply keeps a min() bound on the last
// tile, which executes the same iterations in the same order.
// vectorize / unroll: the loop is cut into whole groups of `factor` iterations, which are split, and a remainder
// that a definition of its own computes (reference: tiramisu_core.cpp:1238-1274 -> separateAndSplit); where the
// loop's bounds are not single affine expressions of the parameters the loop is split as a whole and the inner
// loop keeps a min() bound on the last group.
void computation::separate_and_split(int level, int factor, const std::string &outer, const std::string &inner,
                                     bool &split_applied) {
    isl_set *ts = isl_set_apply(isl_set_copy(iteration_domain), isl_map_copy(schedule));
    const int p = dynamic_pos(level), n = (int)level_names.size();
    isl_set *level_values = isl_set_project_out(isl_set_copy(ts), isl_dim_set, p + 1, 2 * n + 2 - (p + 1));
    level_values = isl_set_project_out(level_values, isl_dim_set, 0, p);
    const bool separable = !single_piece_text(isl_set_dim_max(isl_set_copy(level_values), 0)).empty() &&
                           !single_piece_text(isl_set_dim_min(level_values, 0)).empty() && !fct->backend_option("TIRAMISU_NO_SEPARATION");
    isl_val *mx = isl_set_dim_max_val(isl_set_copy(ts), p);
    isl_val *mn = isl_set_dim_min_val(ts, p);
    long extent = -1;
    if (mx && mn && isl_val_is_int(mx) == isl_bool_true && isl_val_is_int(mn) == isl_bool_true)
        extent = isl_val_get_num_si(mx) - isl_val_get_num_si(mn) + 1;
    isl_val_free(mx);
    isl_val_free(mn);
    split_applied = !(extent > 0 && extent <= factor);
    if (!split_applied) return;
    if (separable) separateAndSplit(level, factor);
    else split(level, factor);
    level_names[level] = outer;
    level_names[level + 1] = inner;
}

void computation::vectorize(var L, int v, var L_outer, var L_inner) {
    int l = get_loop_level_number_from_dimension_name(L.get_name());
    bool applied;
    separate_and_split(l, v, L_outer.get_name(), L_inner.get_name(), applied);
    tag_vector_level(applied ? l + 1 : l, v);
}
void computation::vectorize(var L, int v) {
    vectorize(L, v, var(fct->generate_new_name(L.get_name() + "_vo")), var(fct->generate_new_name(L.get_name() + "_vi")));
}
void computation::unroll(var L, int fac, var L_outer, var L_inner) {
    int l = get_loop_level_number_from_dimension_name(L.get_name());
    bool applied;
    separate_and_split(l, fac, L_outer.get_name(), L_inner.get_name(), applied);
    tag_unroll_level(applied ? l + 1 : l, fac);
}
void computation::unroll(var L, int fac) {
    unroll(L, fac, var(fct->generate_new_name(L.get_name() + "_uo")), var(fct->generate_new_name(L.get_name() + "_ui")));
}

int computation::compute_maximal_AST_depth() { return (int)level_names.size(); }

// ------------------------------------------------------------------ ordering

void computation::after(computation &comp, int level) {
    auto &edges = fct->sched_graph[&comp];
    auto it = edges.find(this);
    if (it != edges.end() && it->second > level) level = it->second;
    edges[this] = level;
    fct->starting_computations.erase(this);
    fct->sched_graph_reversed[this][&comp] = level;
    if (fct->sched_graph_reversed[this].size() > 1)
        ERROR("computation " + name + " has more than one predecessor in the ordering graph", true);
}

void computation::after(computation &comp, var level) {
    after(comp, get_loop_level_number_from_dimension_name(level.get_name()));
}
void computation::before(computation &consumer, var L) { consumer.after(*this, L); }
void computation::before(computation &consumer, int L) { consumer.after(*this, L); }

void computation::between(computation &before_c, int before_l, computation &after_c, int after_l) {
    auto &g = fct->sched_graph;
    if (g[&before_c].count(&after_c)) {
        g[&before_c].erase(&after_c);
        fct->sched_graph_reversed[&after_c].erase(&before_c);
    }
    after(before_c, before_l);
    after_c.after(*this, after_l);
}
void computation::between(computation &before_c, var before_l, computation &after_c, var after_l) {
    int bl = get_loop_level_number_from_dimension_name(before_l.get_name());
    int al = after_c.get_loop_level_number_from_dimension_name(after_l.get_name());
    between(before_c, bl, after_c, al);
}

computation &computation::then(computation &next, var L) { next.after(*this, L); return next; }
computation &computation::then(computation &next, int L) { next.after(*this, L); return next; }

computation *computation::get_predecessor() {
    auto it = fct->sched_graph_reversed.find(this);
    return (it == fct->sched_graph_reversed.end() || it->second.empty()) ? nullptr : it->second.begin()->first;
}

computation *computation::get_successor() {
    auto it = fct->sched_graph.find(this);
    return (it == fct->sched_graph.end() || it->second.empty()) ? nullptr : it->second.begin()->first;
}

// Static dimensions before the fuse level are copied from the predecessor; the one right
// after the fuse level becomes the predecessor's + 10 (reference: tiramisu_core.cpp:2126-2185).
void computation::after_low_level(computation &comp, int level) {
    fct->align_schedules();
    int r = isl_map_dim(schedule, isl_dim_out);
    int last_static = static_pos(level + 1);
    if (last_static >= r) ERROR("after: level " + std::to_string(level) + " is deeper than the schedule of " + name, true);
    for (int pos = 1; pos <= last_static; pos += 2) {
        isl_val *v = isl_map_plain_get_val_if_fixed(comp.schedule, isl_dim_out, pos);
        long order = (v && isl_val_is_int(v) == isl_bool_true) ? isl_val_get_num_si(v) : 0;
        isl_val_free(v);
        if (pos == last_static) order += 10;
        // Replace the constant at this position.
        std::vector<std::string> in, out;
        for (int i = 0; i < r; i++) { in.push_back("x" + std::to_string(i)); out.push_back(in.back()); }
        out[pos] = std::to_string(order);
        apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    }
}

// ------------------------------------------------------------------ GPU mapping

void computation::tag_gpu_block_level(int L0) { fct->add_gpu_block_dimensions(name, L0); }
void computation::tag_gpu_block_level(int L0, int L1) { fct->add_gpu_block_dimensions(name, L0, L1); }
void computation::tag_gpu_block_level(int L0, int L1, int L2) { fct->add_gpu_block_dimensions(name, L0, L1, L2); }
void computation::tag_gpu_thread_level(int L0) { fct->add_gpu_thread_dimensions(name, L0); }
void computation::tag_gpu_thread_level(int L0, int L1) { fct->add_gpu_thread_dimensions(name, L0, L1); }
void computation::tag_gpu_thread_level(int L0, int L1, int L2) { fct->add_gpu_thread_dimensions(name, L0, L1, L2); }

void computation::tag_gpu_level(int L0, int L1) { tag_gpu_block_level(L0); tag_gpu_thread_level(L1); }
void computation::tag_gpu_level(int L0, int L1, int L2, int L3) { tag_gpu_block_level(L0, L1); tag_gpu_thread_level(L2, L3); }
void computation::tag_gpu_level(int L0, int L1, int L2, int L3, int L4, int L5) {
    tag_gpu_block_level(L0, L1, L2);
    tag_gpu_thread_level(L3, L4, L5);
}
void computation::tag_gpu_level(var L0, var L1) {
    auto l = get_loop_level_numbers_from_dimension_names({L0.get_name(), L1.get_name()});
    tag_gpu_level(l[0], l[1]);
}
void computation::tag_gpu_level(var L0, var L1, var L2, var L3) {
    auto l = get_loop_level_numbers_from_dimension_names({L0.get_name(), L1.get_name(), L2.get_name(), L3.get_name()});
    tag_gpu_level(l[0], l[1], l[2], l[3]);
}
void computation::tag_gpu_level(var L0, var L1, var L2, var L3, var L4, var L5) {
    auto l = get_loop_level_numbers_from_dimension_names(
        {L0.get_name(), L1.get_name(), L2.get_name(), L3.get_name(), L4.get_name(), L5.get_name()});
    tag_gpu_level(l[0], l[1], l[2], l[3], l[4], l[5]);
}

void computation::gpu_tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer, var L0_inner,
                           var L1_inner) {
    tile(L0, L1, sizeX, sizeY, L0_outer, L1_outer, L0_inner, L1_inner);
    tag_gpu_level(L0_outer, L1_outer, L0_inner, L1_inner);
    thread_block_shape = {sizeX, sizeY};
}
void computation::gpu_tile(var L0, var L1, int sizeX, int sizeY) {
    auto g = [&](const var &v, const char *s) { return var(fct->generate_new_name(v.get_name() + s)); };
    gpu_tile(L0, L1, sizeX, sizeY, g(L0, "_b"), g(L1, "_b"), g(L0, "_t"), g(L1, "_t"));
}
void computation::gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer, var L1_outer,
                           var L2_outer, var L0_inner, var L1_inner, var L2_inner) {
    tile(L0, L1, L2, sizeX, sizeY, sizeZ, L0_outer, L1_outer, L2_outer, L0_inner, L1_inner, L2_inner);
    tag_gpu_level(L0_outer, L1_outer, L2_outer, L0_inner, L1_inner, L2_inner);
    thread_block_shape = {sizeX, sizeY, sizeZ};
}
void computation::gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ) {
    auto g = [&](const var &v, const char *s) { return var(fct->generate_new_name(v.get_name() + s)); };
    gpu_tile(L0, L1, L2, sizeX, sizeY, sizeZ, g(L0, "_b"), g(L1, "_b"), g(L2, "_b"), g(L0, "_t"), g(L1, "_t"), g(L2, "_t"));
}

// ------------------------------------------------------------------ cache_shared

// The loop-level space of this computation restricted to its first `keep` levels, as an isl set
// string with the level names as dimension names and `tuple` as its name.
static std::string level_space(computation &c, int keep, const std::string &tuple) {
    isl_set *ts = isl_set_apply(isl_set_copy(c.get_iteration_domain()), isl_map_copy(c.get_schedule()));
    int n = (int)c.get_loop_level_names().size();
    // range is [dup, s0, d0, s1, ..., d(n-1), sn]: drop everything but d0..d(keep-1)
    for (int pos = 2 * n + 1; pos >= 0; pos--) {
        bool dynamic = pos >= 2 && pos % 2 == 0;
        int level = (pos - 2) / 2;
        if (!dynamic || level >= keep) ts = isl_set_project_out(ts, isl_dim_set, pos, 1);
    }
    for (int l = 0; l < keep; l++) ts = isl_set_set_dim_name(ts, isl_dim_set, l, c.get_loop_level_names()[l].c_str());
    ts = isl_set_set_tuple_name(ts, tuple.c_str());
    ts = isl_set_coalesce(ts);
    char *str = isl_set_to_str(ts);
    std::string r(str);
    free(str);
    isl_set_free(ts);
    return r;
}

computation *computation::cache_shared(computation &inp, const var &level, const std::vector<int> buffer_shape,
                                       const std::vector<expr> copy_offsets, bool pad_buffer) {
    const size_t nd = inp.iterator_names_.size();
    if (buffer_shape.size() != nd || copy_offsets.size() != nd)
        ERROR("cache_shared: buffer shape and copy offsets must have one entry per dimension of " + inp.get_name(), true);
    const int copy_level = get_loop_level_number_from_dimension_name(level.get_name());
    std::tuple<int, int, int> block_dims(-1, -1, -1), thread_dims(-1, -1, -1);
    for (auto &d : fct->gpu_block_dimensions) if (d.first == name) block_dims = d.second;
    for (auto &d : fct->gpu_thread_dimensions) if (d.first == name) thread_dims = d.second;
    if (std::get<0>(block_dims) == -1) ERROR("cache_shared: " + name + " is not mapped to the GPU", true);
    if (thread_block_shape.empty()) ERROR("cache_shared: " + name + " has no thread block shape (use gpu_tile)", true);

    // LDS buffer; padding the innermost dimension by one element avoids bank conflicts of
    // column accesses (reference: tiramisu_core.cpp:9331-9336)
    const std::string prefix = "_" + name + "_" + inp.get_name();
    std::vector<expr> shape;
    for (int v : buffer_shape) shape.push_back(expr((int32_t)v));
    if (pad_buffer) shape.back() = expr((int32_t)(buffer_shape.back() + 1));
    buffer *shared = new buffer(prefix + "_shared", shape, inp.get_data_type(), a_temporary, fct);
    shared->tag_gpu_shared();

    // reads of inp in this computation now go to the LDS tile: index modulo the tile shape
    std::vector<var> access_vars;
    std::vector<expr> access_exprs;
    for (size_t d = 0; d < nd; d++) {
        var v(inp.iterator_names_[d]);
        access_vars.push_back(var(inp.iterator_names_[d], expr((int32_t)0), expr((int32_t)0x3fffffff)));
        access_exprs.push_back(v % buffer_shape[d]);
    }
    bool saved = global::is_auto_data_mapping_set();
    global::set_auto_data_mapping(false);
    input *new_access = new input(prefix + "_access", access_vars, inp.get_data_type());
    global::set_auto_data_mapping(saved);
    new_access->store_in(shared, access_exprs);
    if (!uncached_expression.is_defined()) uncached_expression = expression;
    set_expression(expression.substitute_access(inp.get_name(), new_access->get_name()));

    int gpu_level = std::get<0>(thread_dims);
    if (std::get<2>(thread_dims) != -1) gpu_level = std::get<2>(thread_dims);
    else if (std::get<1>(thread_dims) != -1) gpu_level = std::get<1>(thread_dims);

    auto map_like_this = [&](computation *c) {
        fct->gpu_block_dimensions.push_back({c->get_name(), block_dims});
        fct->gpu_thread_dimensions.push_back({c->get_name(), thread_dims});
    };

    // declaration of the tile at the beginning of the kernel
    computation *decl = new computation(level_space(*this, gpu_level + 1, prefix + "_dec"), allocate(*shared), true, p_none, fct);
    map_like_this(decl);

    // cooperative copy: ceil(size / threads) iterations per thread
    long size = 1, pool = 1;
    for (int v : buffer_shape) size *= v;
    for (int v : thread_block_shape) pool *= v;
    const std::string iter = prefix + "_copy_iter";
    std::string copy_dom = level_space(*this, copy_level + 1, prefix + "_copy");
    {
        // append the copy iterator with its bounds
        size_t rb = copy_dom.find(']', copy_dom.find(prefix + "_copy["));
        copy_dom.insert(rb, ", " + iter);
        size_t end = copy_dom.rfind('}');
        std::string cond = "0 <= " + iter + " <= " + std::to_string((size - 1) / pool);
        bool has_constraints = copy_dom.find(':') != std::string::npos;
        copy_dom.insert(end, std::string(has_constraints ? " and " : " : ") + cond + " ");
    }
    // linear thread id, slowest thread dimension first (reference: :9376-9422)
    expr tid = var(level_names[std::get<0>(thread_dims)]);
    if (std::get<1>(thread_dims) != -1) tid = tid * thread_block_shape[1] + var(level_names[std::get<1>(thread_dims)]);
    if (std::get<2>(thread_dims) != -1) tid = tid * thread_block_shape[2] + var(level_names[std::get<2>(thread_dims)]);
    expr copy_index = var(iter) * (int32_t)pool + tid;
    std::vector<expr> tile_idx(nd), src_idx(nd);
    long denom = 1;
    for (int d = (int)nd - 1; d >= 0; d--) {
        tile_idx[d] = (denom == 1 ? copy_index : copy_index / (int32_t)denom) % buffer_shape[d];
        src_idx[d] = tile_idx[d] + copy_offsets[d];
        denom *= buffer_shape[d];
    }
    computation *copy = new computation(copy_dom, expr(o_access, inp.get_name(), src_idx, inp.get_data_type()), true,
                                        inp.get_data_type(), fct);
    copy->store_in(shared, tile_idx);
    if (size % pool != 0) copy->add_predicate(copy_index < (int32_t)size);
    map_like_this(copy);

    // barriers around the copy
    computation *sync1 = new computation(level_space(*this, copy_level + 1, prefix + "_sync1"), tiramisu::sync(), true, p_none, fct);
    computation *sync2 = new computation(level_space(*this, copy_level + 1, prefix + "_sync2"), tiramisu::sync(), true, p_none, fct);
    map_like_this(sync1);
    map_like_this(sync2);

    // order: [...] -> sync1 -> copy -> sync2 -> first computation at the copy level
    // (reference: :9479-9515)
    {
        computation *curr = this, *pred = curr->get_predecessor();
        while (pred != nullptr && fct->sched_graph[pred][curr] >= copy_level) {
            curr = pred;
            pred = curr->get_predecessor();
        }
        if (pred != nullptr) sync1->between(*pred, fct->sched_graph[pred][curr], *curr, copy_level);
        else sync1->before(*curr, copy_level);
        sync2->between(*sync1, copy_level, *curr, copy_level);
        copy->between(*sync1, copy_level, *sync2, copy_level);
    }
    {
        computation *curr = this, *pred = curr->get_predecessor();
        while (pred != nullptr && fct->sched_graph[pred][curr] >= gpu_level) {
            curr = pred;
            pred = curr->get_predecessor();
        }
        if (pred != nullptr) decl->between(*pred, fct->sched_graph[pred][curr], *curr, gpu_level);
        else decl->before(*curr, gpu_level);
    }
    shared_cache rec;
    rec.input = inp.get_name();
    rec.access = new_access->get_name();
    rec.shape = buffer_shape;
    rec.offsets = copy_offsets;
    rec.copy_level = copy_level;
    rec.apparatus = {decl, copy, sync1, sync2};
    for (computation *c : rec.apparatus) c->cache_consumer = this;
    shared_caches.push_back(rec);
    return new_access;
}

bool computation::shared_caches_cover_reads() const {
    if (shared_caches.empty()) return true;
    if (!uncached_expression.is_defined() || predicate.is_defined()) return false;
    const int nl = (int)level_names.size();
    // iteration-domain dimensions are renamed: a loop level may carry an iterator's name with another value
    std::map<std::string, std::string> rename;
    std::vector<std::string> dom_names;
    for (size_t d = 0; d < iterator_names_.size(); d++) {
        dom_names.push_back("_it" + std::to_string(d));
        rename[iterator_names_[d]] = dom_names.back();
    }
    std::map<std::string, expr> rename_subs;
    for (auto &r : rename) rename_subs[r.first] = expr(var(global::get_loop_iterator_data_type(), r.second));
    auto renamed = [&](const expr &e) { return e.substitute(rename_subs); };
    std::vector<std::string> range = {"_dup"};
    for (int l = 0; l <= nl; l++) {
        range.push_back("_s" + std::to_string(l));
        if (l < nl) range.push_back(level_names[l]);
    }
    std::set<std::string> params;
    for (int i = 0; i < (int)isl_set_dim(iteration_domain, isl_dim_param); i++)
        params.insert(isl_set_get_dim_name(iteration_domain, isl_dim_param, i));
    std::vector<std::string> bad;
    for (const shared_cache &sc : shared_caches) {
        std::vector<std::vector<expr>> reads;
        uncached_expression.visit([&](const expr &x) {
            if (x.get_expr_type() == e_op && x.get_op_type() == o_access && x.get_name() == sc.input) reads.push_back(x.get_access());
        });
        if (reads.empty()) return false;
        for (size_t d = 0; d < sc.shape.size(); d++) {
            // the tile origin may depend on the loop levels down to the copy level only
            bool names_ok = true;
            sc.offsets[d].visit([&](const expr &x) {
                if (x.get_expr_type() != e_var) return;
                auto it = std::find(level_names.begin(), level_names.end(), x.get_name());
                if (it == level_names.end() ? !params.count(x.get_name()) : (it - level_names.begin()) > sc.copy_level) names_ok = false;
            });
            if (!names_ok) return false;
            bool ok = true;
            const std::string off = expr_to_isl_str(sc.offsets[d], ok), n = std::to_string(sc.shape[d]);
            if (!ok) return false;
            bad.push_back("(" + off + ") mod " + n + " != 0");
            for (auto &idx : reads) {
                if (idx.size() != sc.shape.size()) return false;
                const std::string at = expr_to_isl_str(renamed(idx[d]), ok);
                if (!ok) return false;
                bad.push_back(at + " < " + off);
                bad.push_back(at + " >= " + off + " + " + n);
            }
        }
    }
    std::vector<std::string> pv(params.begin(), params.end());
    const std::string text = params_prefix(pv) + "{ " + name + "[" + join(dom_names, ", ") + "] -> [" + join(range, ", ") + "] : " +
                             join(bad, " or ") + " }";
    isl_map *violations = isl_map_read_from_str(ctx, text.c_str());
    if (!violations) return false;
    isl_set *dom = isl_set_copy(iteration_domain);
    if (fct->get_program_context()) dom = isl_set_intersect_params(dom, isl_set_copy(fct->get_program_context()));
    isl_map *sched = isl_map_intersect_domain(isl_map_copy(schedule), dom);
    violations = isl_map_intersect(sched, violations);   // positional: dimension names play no part
    const bool covered = isl_map_is_empty(violations) == isl_bool_true;
    isl_map_free(violations);
    return covered;
}

// ------------------------------------------------------------------ separation, duplicates, compute_at, storage folding

static std::string function_params(function *f) { return params_prefix(f->get_invariant_names()); }

// the time-space tuple of a schedule with n levels as variables x0 ... x(2n+1)
static std::string time_space_tuple(int levels) {
    std::vector<std::string> v;
    range_vars(levels, v);
    return "[" + join(v, ",") + "]";
}

bool computation::executed_range(int dim, long &lowest, long &highest) const {
    isl_set *points = isl_map_domain(isl_map_intersect_domain(isl_map_copy(schedule), isl_set_copy(iteration_domain)));
    bool ok = isl_set_is_empty(points) != isl_bool_true && dim >= 0 && dim < (int)isl_set_dim(points, isl_dim_set);
    if (ok) {
        isl_val *a = isl_set_dim_min_val(isl_set_copy(points), dim), *b = isl_set_dim_max_val(isl_set_copy(points), dim);
        ok = a && b && isl_val_is_int(a) == isl_bool_true && isl_val_is_int(b) == isl_bool_true;
        if (ok) { lowest = isl_val_get_num_si(a); highest = isl_val_get_num_si(b); }
        isl_val_free(a);
        isl_val_free(b);
    }
    isl_set_free(points);
    return ok;
}

void buffer::set_dim_size(int dim, int size) {
    if (dim < 0 || dim >= (int)dim_sizes.size() || size <= 0) ERROR("set_dim_size: bad dimension or size for buffer " + name, true);
    dim_sizes[dim] = expr((int32_t)size);
}

// A copy of this computation under another name: same iteration domain, expression, schedule, level names and
// data mapping; a definition of the same first definition, so accesses to it keep reading through that one.
computation *computation::copy_as(const std::string &new_name) {
    isl_set *dom = isl_set_set_tuple_name(isl_set_copy(iteration_domain), new_name.c_str());
    char *text = isl_set_to_str(dom);
    computation *c = new computation(std::string(text), expression, schedule_this, data_type, fct);
    free(text);
    isl_set_free(dom);
    c->iterator_names_ = iterator_names_;
    c->level_names = level_names;
    c->declared_vars = declared_vars;
    if (c->schedule) isl_map_free(c->schedule);
    c->schedule = isl_map_set_tuple_name(isl_map_copy(schedule), isl_dim_in, new_name.c_str());
    if (access) c->access = isl_map_set_tuple_name(isl_map_copy(access), isl_dim_in, new_name.c_str());
    c->predicate = predicate;
    c->associated_let_stmts = associated_let_stmts;
    c->is_let = is_let;
    c->inline_ = inline_;
    c->first_definition = get_first_definition();
    return c;
}

// Cut at loop level `dim`: this computation keeps the time-space points with x(dim) < bound, a new definition
// takes x(dim) >= bound and runs after this one at that level.
void computation::separate_by_text(int dim, const std::string &bound, const std::string &params) {
    const int n = (int)level_names.size();
    if (dim < 0 || dim >= n) ERROR("separate: level out of range for " + name, true);
    const std::string x = "x" + std::to_string(dynamic_pos(dim));
    const std::string full = params + "{ " + time_space_tuple(n) + " : " + x + " < " + bound + " }";
    const std::string rest = params + "{ " + time_space_tuple(n) + " : " + x + " >= " + bound + " }";
    isl_set *rest_set = isl_set_read_from_str(ctx, rest.c_str());
    if (!rest_set) ERROR("separate: cannot parse " + rest, true);
    isl_map *there = isl_map_intersect_range(isl_map_intersect_domain(isl_map_copy(schedule), isl_set_copy(iteration_domain)), rest_set);
    const bool empty = isl_map_is_empty(there) == isl_bool_true;
    isl_map_free(there);
    if (!empty) {
        computation *first = get_first_definition();
        computation *c = copy_as("_" + first->name + "_update_" + std::to_string(first->updates.size() + 1));
        first->updates.push_back(c);
        c->add_schedule_constraint("", rest);
        c->after(*this, dim);
    }
    add_schedule_constraint("", full);
}

void computation::separate(int dim, expr N, int v, expr lower_bound) {
    bool ok = true;
    const std::string n_text = expr_to_isl_str(N, ok), lower = expr_to_isl_str(lower_bound, ok);
    if (!ok || v < 1) ERROR("separate: the loop extent and lower bound must be affine, the factor positive (" + name + ")", true);
    separate_by_text(dim, "(" + std::to_string(v) + " * floor((" + n_text + ") / " + std::to_string(v) + ") + (" + lower + "))", function_params(fct));
}

void computation::separate_at(var level, std::vector<expr> separate_points, expr max) {
    if (separate_points.empty()) ERROR("separate_at: no separation point given for " + name, true);
    const int dim = get_loop_level_number_from_dimension_name(level.get_name());
    const int n = (int)level_names.size();
    const std::string x = "x" + std::to_string(dynamic_pos(dim)), params = function_params(fct);
    bool ok = true;
    std::vector<std::string> cut;
    for (auto &pt : separate_points) cut.push_back("(" + expr_to_isl_str(pt, ok) + ")");
    cut.push_back("(" + expr_to_isl_str(max, ok) + ")");
    if (!ok) ERROR("separate_at: separation points must be affine (" + name + ")", true);
    computation *first = get_first_definition();
    computation *previous = this;
    for (size_t k = 0; k + 1 < cut.size(); k++) {
        const std::string piece = params + "{ " + time_space_tuple(n) + " : " + x + " >= " + cut[k] + " and " + x + " < " + cut[k + 1] + " }";
        isl_set *piece_set = isl_set_read_from_str(ctx, piece.c_str());
        if (!piece_set) ERROR("separate_at: cannot parse " + piece, true);
        isl_map *there = isl_map_intersect_range(isl_map_intersect_domain(isl_map_copy(schedule), isl_set_copy(iteration_domain)), piece_set);
        const bool empty = isl_map_is_empty(there) == isl_bool_true;
        isl_map_free(there);
        if (empty) continue;
        computation *c = copy_as("_" + first->name + "_update_" + std::to_string(first->updates.size() + 1));
        first->updates.push_back(c);
        c->add_schedule_constraint("", piece);
        c->after(*previous, dim);
        previous = c;
    }
    add_schedule_constraint("", params + "{ " + time_space_tuple(n) + " : " + x + " < " + cut[0] + " }");
}

// "(text)" of the single affine piece of a bound, empty when the bound is piecewise
static std::string single_piece_text(isl_pw_aff *pa) {
    std::string out;
    if (pa && isl_pw_aff_n_piece(pa) == 1) {
        char *t = isl_pw_aff_to_str(pa);          // "[N] -> { [(-1 + N)] }"
        std::string s = t ? t : "";
        free(t);
        const size_t a = s.find("[("), b = s.rfind(")]");
        if (a != std::string::npos && b != std::string::npos && b > a && s.find(" : ", a) == std::string::npos) out = s.substr(a + 1, b - a);
    }
    if (pa) isl_pw_aff_free(pa);
    return out;
}

void computation::split_with_lower_bound(int L0, int sizeX, std::string lower_bound) {
    const int n = (int)level_names.size();
    if (L0 < 0 || L0 >= n) ERROR("split: level out of range for " + name, true);
    if (sizeX < 1) ERROR("split: factor must be positive", true);
    std::vector<std::string> in, out;
    range_vars(n, in);
    const std::string d = "(" + in[dynamic_pos(L0)] + " - (" + lower_bound + "))", f = std::to_string(sizeX);
    for (int i = 0; i < (int)in.size(); i++) {
        if (i != dynamic_pos(L0)) { out.push_back(in[i]); continue; }
        out.push_back("floor(" + d + " / " + f + ")");
        out.push_back("0");
        out.push_back(d + " mod " + f);
    }
    apply_on_range(function_params(fct) + "{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    level_names.insert(level_names.begin() + L0 + 1, fct->generate_new_name(level_names[L0] + "_in"));
}

bool computation::separateAndSplit(int L0, int v) {
    const int n = (int)level_names.size();
    if (L0 < 0 || L0 >= n) ERROR("separateAndSplit: level out of range for " + name, true);
    isl_set *ts = isl_set_apply(isl_set_copy(iteration_domain), isl_map_copy(schedule));
    const int p = dynamic_pos(L0);
    // a loop of at most v iterations stays as it is
    isl_val *mx = isl_set_dim_max_val(isl_set_copy(ts), p), *mn = isl_set_dim_min_val(isl_set_copy(ts), p);
    long extent = -1;
    if (mx && mn && isl_val_is_int(mx) == isl_bool_true && isl_val_is_int(mn) == isl_bool_true) extent = isl_val_get_num_si(mx) - isl_val_get_num_si(mn) + 1;
    isl_val_free(mx);
    isl_val_free(mn);
    if (extent > 0 && extent <= v) { isl_set_free(ts); return false; }
    // bounds of the level in terms of the parameters alone
    isl_set *level_values = isl_set_project_out(isl_set_copy(ts), isl_dim_set, p + 1, 2 * n + 2 - (p + 1));
    level_values = isl_set_project_out(level_values, isl_dim_set, 0, p);
    const std::string upper = single_piece_text(isl_set_dim_max(isl_set_copy(level_values), 0));
    const std::string lower = single_piece_text(isl_set_dim_min(level_values, 0));
    isl_set_free(ts);
    if (upper.empty() || lower.empty()) ERROR("separateAndSplit: the bounds of level " + level_names[L0] + " of " + name + " are not single affine expressions of the parameters", true);
    const std::string count = "(" + upper + " - " + lower + " + 1)", f = std::to_string(v);
    std::vector<std::string> params;
    for (int i = 0; i < (int)isl_map_dim(schedule, isl_dim_param); i++) params.push_back(isl_map_get_dim_name(schedule, isl_dim_param, i));
    for (auto &nm : fct->get_invariant_names()) if (std::find(params.begin(), params.end(), nm) == params.end()) params.push_back(nm);
    separate_by_text(L0, "(" + f + " * floor(" + count + " / " + f + ") + " + lower + ")", params_prefix(params));
    split_with_lower_bound(L0, v, lower);
    return true;
}

bool computation::separateAndSplit(var L0, int sizeX, var L0_outer, var L0_inner) {
    const int l = get_loop_level_number_from_dimension_name(L0.get_name());
    assert_names_not_assigned({L0_outer.get_name(), L0_inner.get_name()});
    const bool split_happened = separateAndSplit(l, sizeX);
    level_names[l] = L0_outer.get_name();
    if (split_happened) level_names[l + 1] = L0_inner.get_name();
    return split_happened;
}

bool computation::separateAndSplit(var L0, int sizeX) {
    return separateAndSplit(L0, sizeX, var(fct->generate_new_name(L0.get_name() + "_so")), var(fct->generate_new_name(L0.get_name() + "_si")));
}

computation *computation::duplicate(std::string domain_constraints, std::string range_constraints) {
    fct->align_schedules();
    computation *first = get_first_definition();
    computation *c = copy_as("_" + first->name + "_dup_" + std::to_string(first->duplicates.size() + 1));
    first->duplicates.push_back(c);
    if (!domain_constraints.empty()) {
        isl_set *d = isl_set_read_from_str(ctx, domain_constraints.c_str());
        if (!d) ERROR("duplicate: cannot parse " + domain_constraints, true);
        d = isl_set_set_tuple_name(d, c->name.c_str());
        c->schedule = isl_map_intersect_domain(c->schedule, d);
    }
    c->add_schedule_constraint("", range_constraints);
    // the duplicate's number goes into the first time-space dimension
    std::vector<std::string> in, out;
    range_vars((int)c->level_names.size(), in);
    out = in;
    out[0] = std::to_string(first->duplicates.size());
    c->apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    return c;
}

computation *computation::select(int duplicate_id) {
    computation *first = get_first_definition();
    if (duplicate_id == 0) return this;
    if (duplicate_id < 0 || duplicate_id > (int)first->duplicates.size()) ERROR("select: " + name + " has no duplicate number " + std::to_string(duplicate_id), true);
    return first->duplicates[duplicate_id - 1];
}

// { consumer[iterators] -> producer[indices] } for every read of `producer` in the consumer's expression and predicate
isl_map *reads_of(computation &consumer, computation &producer, bool within_producer_domain, bool any_where_not_affine) {
    function *f = consumer.get_function();
    const std::string wanted = producer.get_first_definition()->get_name();
    std::vector<std::string> pieces;
    bool ok = true;
    int free_dimensions = 0;
    auto collect = [&](const expr &e) {
        if (!e.is_defined()) return;
        e.visit([&](const expr &x) {
            if (x.get_expr_type() != e_op || x.get_op_type() != o_access || x.get_name() != wanted) return;
            std::vector<std::string> idx;
            for (auto &i : x.get_access()) {
                bool affine = true;
                std::string text = expr_to_isl_str(i, affine);
                // an index looked up in a table (or otherwise not affine) may be anything: a free dimension
                if (!affine && any_where_not_affine) text = "_any" + std::to_string(free_dimensions++);
                else ok = ok && affine;
                idx.push_back(text);
            }
            pieces.push_back(consumer.get_name() + "[" + join(consumer.get_iteration_domain_dimension_names(), ",") + "] -> " + producer.get_name() + "[" + join(idx, ",") + "]");
        });
    };
    collect(consumer.get_expr());
    collect(consumer.get_predicate());
    if (!ok) ERROR("an index of " + wanted + " in " + consumer.get_name() + " is not affine", true);
    if (pieces.empty()) return nullptr;
    isl_map *all = nullptr;
    for (auto &pc : pieces) {
        isl_map *m = isl_map_read_from_str(f->get_isl_ctx(), (function_params(f) + "{ " + pc + " }").c_str());
        if (!m) ERROR("cannot parse read relation " + pc, true);
        all = all ? isl_map_union(all, m) : m;
    }
    all = isl_map_intersect_domain(all, isl_set_copy(consumer.get_iteration_domain()));
    return within_producer_domain ? isl_map_intersect_range(all, isl_set_copy(producer.get_iteration_domain())) : all;
}

std::vector<computation *> function::get_live_out_computations() {
    std::vector<computation *> out;
    for (auto c : body) {
        if (c->is_inline_computation() || !c->get_expr().is_defined() && !c->should_schedule_this_computation()) continue;
        const std::string nm = c->get_first_definition()->get_name();
        bool is_read = false;
        for (auto k : body) {
            if (k->get_first_definition() == c->get_first_definition()) continue;
            for (const expr *e : {&k->get_expr(), &k->get_predicate()})
                if (e->is_defined()) e->visit([&](const expr &x) { if (x.get_expr_type() == e_op && x.get_op_type() == o_access && x.get_name() == nm) is_read = true; });
        }
        if (!is_read) out.push_back(c);
    }
    return out;
}

void function::compute_bounds() {
    std::map<computation *, isl_set *> frontier;
    for (auto c : get_live_out_computations()) frontier[c] = isl_set_copy(c->get_iteration_domain());
    for (size_t round = 0; round <= body.size() && !frontier.empty(); round++) {
        std::map<computation *, isl_set *> next;
        for (auto &fr : frontier) {
            for (auto p : body) {
                if (p->get_first_definition() == fr.first->get_first_definition()) continue;       // a computation reading itself adds nothing
                if (!p->is_first_definition() || !p->get_updates().empty()) continue;               // several definitions: the user's domains stay
                isl_map *m = reads_of(*fr.first, *p, false);
                if (!m) continue;
                isl_set *needed = isl_set_apply(isl_set_copy(fr.second), m);
                if (isl_set_is_empty(needed) == isl_bool_true) { isl_set_free(needed); continue; }
                next[p] = next.count(p) ? isl_set_union(next[p], needed) : needed;
            }
            isl_set_free(fr.second);
        }
        for (auto &nx : next) {
            computation *p = nx.first;
            isl_set *dom = isl_set_plain_is_universe(p->iteration_domain) == isl_bool_true
                               ? isl_set_copy(nx.second) : isl_set_union(isl_set_copy(p->iteration_domain), isl_set_copy(nx.second));
            dom = isl_set_coalesce(dom);
            dom = isl_set_set_tuple_name(dom, p->name.c_str());
            for (size_t d = 0; d < p->iterator_names_.size(); d++) dom = isl_set_set_dim_name(dom, isl_dim_set, (unsigned)d, p->iterator_names_[d].c_str());
            isl_set_free(p->iteration_domain);
            p->iteration_domain = dom;
        }
        frontier = next;
    }
    for (auto &fr : frontier) isl_set_free(fr.second);
}

void computation::compute_at(computation &consumer, var L) {
    compute_at(consumer, consumer.get_loop_level_number_from_dimension_name(L.get_name()));
}

void computation::compute_at(computation &consumer, int L) {
    fct->align_schedules();
    const int n = (int)isl_map_dim(schedule, isl_dim_out);                  // 2 * levels + 2, the same for both now
    if (L < root_dimension || dynamic_pos(L) >= n) ERROR("compute_at: level out of range for " + consumer.name, true);
    // `first`, the head of the chain that ends in this computation, goes right before the consumer: behind the
    // consumer's present predecessor if it has one
    auto chain_before_consumer = [&](computation *first) {
        computation *q = consumer.get_predecessor();
        if (q && q != this && q != first) {
            const int level_q = fct->sched_graph[q][&consumer];
            fct->sched_graph[q].erase(&consumer);
            fct->sched_graph_reversed[&consumer].erase(q);
            first->after(*q, level_q);
        }
        consumer.after(*this, L);
    };
    isl_map *reads = reads_of(consumer, *this);
    if (!reads || L == root_dimension) {
        // nothing read (or the whole nests one after the other): ordering only
        if (reads) isl_map_free(reads);
        chain_before_consumer(this);
        return;
    }
    // reads, consumer and producer in time-space coordinates; the loops down to L pinned to parameters _T0 ... _TL
    reads = isl_map_apply_range(isl_map_apply_domain(reads, isl_map_copy(consumer.schedule)), isl_map_copy(schedule));
    std::vector<std::string> vars, t_names, pins, distances;
    for (int i = 0; i < n; i++) vars.push_back("x" + std::to_string(i));
    for (int i = 0; i <= L; i++) {
        t_names.push_back("_T" + std::to_string(i));
        pins.push_back(vars[dynamic_pos(i)] + " = " + t_names.back());
        distances.push_back(vars[dynamic_pos(i)] + " - " + t_names.back());
    }
    const std::string t_params = "[" + join(t_names, ",") + "] -> ";
    isl_set *pin = isl_set_read_from_str(ctx, (t_params + "{ [" + join(vars, ",") + "] : " + join(pins, " and ") + " }").c_str());
    isl_set *consumer_ts = isl_set_intersect(isl_set_apply(isl_set_copy(consumer.iteration_domain), isl_map_copy(consumer.schedule)), isl_set_copy(pin));
    isl_set *produced = isl_set_intersect(isl_set_apply(isl_set_copy(iteration_domain), isl_map_copy(schedule)), pin);
    isl_set *needed = isl_set_apply(consumer_ts, reads);
    isl_set *missing = isl_set_coalesce(isl_set_subtract(needed, produced));
    if (isl_set_is_empty(missing) == isl_bool_true) {
        isl_set_free(missing);
        chain_before_consumer(this);
        return;
    }
    // How far, per level, the missing points lie from the iteration that needs them: the set of distance vectors
    // (x(level) - _T(level)) must be a few constant vectors.
    isl_set *vectors = isl_set_apply(isl_set_copy(missing),
                                     isl_map_read_from_str(ctx, (t_params + "{ [" + join(vars, ",") + "] -> [" + join(distances, ",") + "] }").c_str()));
    vectors = isl_set_project_out(vectors, isl_dim_param, 0, isl_set_dim(vectors, isl_dim_param));
    std::vector<std::vector<int>> found;
    while (isl_set_is_empty(vectors) != isl_bool_true) {
        if (found.size() == 32) ERROR("compute_at: what " + consumer.name + " reads of " + name + " outside its own iterations is not at a few fixed distances", true);
        isl_set *pt = isl_set_lexmin(isl_set_copy(vectors));
        std::vector<int> v;
        for (int i = 0; i <= L; i++) {
            isl_val *c = isl_set_plain_get_val_if_fixed(pt, isl_dim_set, i);
            if (!c || isl_val_is_int(c) != isl_bool_true) ERROR("compute_at: what " + consumer.name + " reads of " + name + " outside its own iterations is not at fixed distances", true);
            v.push_back((int)isl_val_get_num_si(c));
            isl_val_free(c);
        }
        found.push_back(v);
        vectors = isl_set_subtract(vectors, pt);
    }
    isl_set_free(vectors);
    // One duplicate computes every missing point, once, early enough for all its readers: at the largest distance
    // per level (a point read from distances c1 and c2 is computed at its own time minus max(c1, c2), which is
    // not later than either reader).  The buffer keeps it for the later readers.
    std::vector<int> farthest = found[0];
    for (auto &v : found)
        for (int i = 0; i <= L; i++) farthest[i] = std::max(farthest[i], v[i]);
    for (auto &t : t_names)
        for (int i = 0; i < (int)isl_set_dim(missing, isl_dim_param); i++)
            if (t == isl_set_get_dim_name(missing, isl_dim_param, i)) { missing = isl_set_project_out(missing, isl_dim_param, i, 1); break; }
    char *text = isl_set_to_str(missing);
    computation *redundant = duplicate("", text);
    free(text);
    for (int i = 0; i <= L; i++)
        if (farthest[i] != 0) redundant->shift(i, -farthest[i]);
    after(*redundant, L);
    computation *head = redundant;
    isl_set_free(missing);
    chain_before_consumer(head);
}

void computation::storage_fold(var L0, int factor) {
    if (!access) ERROR("storage_fold: " + name + " has no data mapping yet", true);
    if (factor < 1) ERROR("storage_fold: factor must be positive", true);
    const int d = get_loop_level_number_from_dimension_name(L0.get_name());
    const int n = (int)isl_map_dim(access, isl_dim_out);
    if (d < 0 || d >= n) ERROR("storage_fold: " + L0.get_name() + " is not a dimension of the buffer of " + name, true);
    buffer *b = get_buffer();
    b->set_dim_size(d, factor);
    std::vector<std::string> in, out;
    for (int i = 0; i < n; i++) {
        in.push_back("o" + std::to_string(i));
        out.push_back(i == d ? in.back() + " mod " + std::to_string(factor) : in.back());
    }
    const std::string bn = b->get_name();
    isl_map *fold = isl_map_read_from_str(ctx, ("{ " + bn + "[" + join(in, ",") + "] -> " + bn + "[" + join(out, ",") + "] }").c_str());
    // every definition and duplicate of this computation that stores in the buffer stores folded: the buffer has
    // shrunk for all of them
    computation *first = get_first_definition();
    std::vector<computation *> all{first};
    all.insert(all.end(), first->updates.begin(), first->updates.end());
    all.insert(all.end(), first->duplicates.begin(), first->duplicates.end());
    for (auto c : all)
        if (c->access && isl_map_get_tuple_name(c->access, isl_dim_out) == bn) c->access = isl_map_apply_range(c->access, isl_map_copy(fold));
    isl_map_free(fold);
}

void computation::gen_time_space_domain() {
    if (time_space_domain) isl_set_free(time_space_domain);
    isl_set *d = isl_set_copy(iteration_domain);
    if (fct->get_program_context())
        d = isl_set_intersect_params(d, isl_set_copy(fct->get_program_context()));
    time_space_domain = isl_set_apply(d, isl_map_copy(schedule));
}

// ------------------------------------------------------------------ input / constant

static std::string fresh_input_name() {
    static int n = 0;
    return "_input" + std::to_string(n++);
}

input::input(std::string nm, std::vector<var> iterator_variables, primitive_t t) {
    fct = global::get_implicit_function();
    if (!fct) ERROR("call tiramisu::init() first", true);
    declared_vars = iterator_variables;
    init_computation(construct_iteration_domain(nm, iterator_variables), fct, expr(), false, t);
    if (global::is_auto_data_mapping_set()) allocate_and_map_buffer_automatically(a_input);
}

input::input(std::vector<var> iterator_variables, primitive_t t) : input(fresh_input_name(), iterator_variables, t) {}

view::view(std::string nm, std::vector<var> iterator_variables, primitive_t t) {
    fct = global::get_implicit_function();
    if (!fct) ERROR("call tiramisu::init() first", true);
    declared_vars = iterator_variables;
    init_computation(construct_iteration_domain(nm, iterator_variables), fct, expr(), false, t);
}

static std::vector<var> vars_from_names_sizes(const std::vector<std::string> &names, const std::vector<expr> &sizes) {
    if (names.size() != sizes.size()) ERROR("input: as many dimension names as sizes are needed", true);
    std::vector<var> v;
    for (size_t i = 0; i < names.size(); i++) v.push_back(var(names[i], expr((int32_t)0), sizes[i]));
    return v;
}

input::input(std::string nm, std::vector<std::string> dimension_names, std::vector<expr> dimension_sizes, primitive_t t)
    : input(nm, vars_from_names_sizes(dimension_names, dimension_sizes), t) {}

std::vector<var> Input::iterators_from_size_expressions(std::vector<expr> sizes) {
    std::vector<var> v;
    for (size_t i = 0; i < sizes.size(); i++) v.push_back(var("_in" + std::to_string(i), expr((int32_t)0), sizes[i]));
    return v;
}
Input::Input(std::string nm, std::vector<expr> sizes, primitive_t t) : input(nm, iterators_from_size_expressions(sizes), t) {}

constant::constant(std::string param_name, const expr &param_expr, primitive_t t, bool function_wide,
                   computation *with_computation, int at_loop_level, function *func) {
    if (!func) func = global::get_implicit_function();
    if (!func) ERROR("call tiramisu::init() first", true);
    if (function_wide != (with_computation == nullptr))
        ERROR("constant " + param_name + ": give a computation exactly when the constant is not function-wide", true);
    if (!function_wide) {
        // A scalar recomputed inside the loop nest of `with_computation`, right before it at loop
        // level `at_loop_level`: its iteration domain is the consumer's projected onto the loops
        // down to that level (reference: tiramisu_core.cpp:8094-8136).
        isl_set *iter = isl_set_copy(with_computation->get_iteration_domain());
        const int keep = at_loop_level + 1, n = isl_set_dim(iter, isl_dim_set);
        if (at_loop_level < computation::root_dimension || keep > n)
            ERROR("constant " + param_name + ": loop level out of range", true);
        iter = isl_set_project_out(iter, isl_dim_set, keep, n - keep);
        iter = isl_set_set_tuple_name(iter, param_name.c_str());
        char *str = isl_set_to_str(iter);
        const std::string domain = str;
        free(str);
        isl_set_free(iter);
        init_computation(domain, func, param_expr, true, t);
        is_let = true;
        if (keep == 0) {
            before(*with_computation, computation::root_dimension);
        } else if (computation *pred = with_computation->get_predecessor()) {
            // keep the consumer's place in the order: predecessor, then this, then the consumer
            const int fused = func->sched_graph[pred][with_computation];
            between(*pred, fused, *with_computation, at_loop_level);
        } else {
            before(*with_computation, at_loop_level);
        }
        return;
    }
    fct = func;
    ctx = fct->get_isl_ctx();
    name = param_name;
    expression = param_expr;
    data_type = t;
    is_let = true;
    schedule_this = false;
    iteration_domain = isl_set_read_from_str(ctx, ("{ " + param_name + "[0] }").c_str());
    iterator_names_ = {"_zero"};
    level_names = iterator_names_;
    set_identity_schedule();
    fct->add_invariant(this);
}

constant::constant(std::string param_name, const expr &param_expr)
    : constant(param_name, param_expr, param_expr.get_data_type(), true, nullptr, 0, global::get_implicit_function()) {}
constant::constant(std::string param_name, const expr &param_expr, primitive_t t, function *func)
    : constant(param_name, param_expr, t, true, nullptr, 0, func) {}

constant::operator expr() { return var(data_type, name); }

// ------------------------------------------------------------------ block

block::block(const std::vector<computation *> c) : children(c) {}

#define FORALL(call) do { for (auto c : children) c->call; } while (0)
void block::gpu_tile(var L0, var L1, int X, int Y) {
    // All children must get the same generated names.
    function *f = children.empty() ? nullptr : children[0]->get_function();
    auto g = [&](const var &v, const char *s) { return var(f->generate_new_name(v.get_name() + s)); };
    gpu_tile(L0, L1, X, Y, g(L0, "_b"), g(L1, "_b"), g(L0, "_t"), g(L1, "_t"));
}
void block::gpu_tile(var L0, var L1, int X, int Y, var a, var b, var c_, var d) { FORALL(gpu_tile(L0, L1, X, Y, a, b, c_, d)); }
void block::gpu_tile(var L0, var L1, var L2, int X, int Y, int Z) {
    function *f = children.empty() ? nullptr : children[0]->get_function();
    auto g = [&](const var &v, const char *s) { return var(f->generate_new_name(v.get_name() + s)); };
    gpu_tile(L0, L1, L2, X, Y, Z, g(L0, "_b"), g(L1, "_b"), g(L2, "_b"), g(L0, "_t"), g(L1, "_t"), g(L2, "_t"));
}
void block::gpu_tile(var L0, var L1, var L2, int X, int Y, int Z, var a, var b, var c_, var d, var e, var f) {
    FORALL(gpu_tile(L0, L1, L2, X, Y, Z, a, b, c_, d, e, f));
}
void block::interchange(var L0, var L1) { FORALL(interchange(L0, L1)); }
void block::interchange(int L0, int L1) { FORALL(interchange(L0, L1)); }
void block::parallelize(var L) { FORALL(parallelize(L)); }
void block::shift(var L0, int n) { FORALL(shift(L0, n)); }
void block::skew(var i, var j, int f, var ni, var nj) { FORALL(skew(i, j, f, ni, nj)); }
void block::split(var L0, int X) {
    function *f = children[0]->get_function();
    split(L0, X, var(f->generate_new_name(L0.get_name() + "_o")), var(f->generate_new_name(L0.get_name() + "_i")));
}
void block::split(var L0, int X, var o, var i) { FORALL(split(L0, X, o, i)); }
void block::split(int L0, int X) { FORALL(split(L0, X)); }
void block::tile(var L0, var L1, int X, int Y) {
    function *f = children[0]->get_function();
    auto g = [&](const var &v, const char *s) { return var(f->generate_new_name(v.get_name() + s)); };
    tile(L0, L1, X, Y, g(L0, "_o"), g(L1, "_o"), g(L0, "_i"), g(L1, "_i"));
}
void block::tile(var L0, var L1, int X, int Y, var a, var b, var c_, var d) { FORALL(tile(L0, L1, X, Y, a, b, c_, d)); }
void block::tile(var L0, var L1, var L2, int X, int Y, int Z) {
    function *f = children[0]->get_function();
    auto g = [&](const var &v, const char *s) { return var(f->generate_new_name(v.get_name() + s)); };
    tile(L0, L1, L2, X, Y, Z, g(L0, "_o"), g(L1, "_o"), g(L2, "_o"), g(L0, "_i"), g(L1, "_i"), g(L2, "_i"));
}
void block::tile(var L0, var L1, var L2, int X, int Y, int Z, var a, var b, var c_, var d, var e, var f) {
    FORALL(tile(L0, L1, L2, X, Y, Z, a, b, c_, d, e, f));
}
void block::tile(int L0, int L1, int X, int Y) { FORALL(tile(L0, L1, X, Y)); }
void block::tile(int L0, int L1, int L2, int X, int Y, int Z) { FORALL(tile(L0, L1, L2, X, Y, Z)); }
void block::unroll(var L, int fac) {
    function *f = children[0]->get_function();
    unroll(L, fac, var(f->generate_new_name(L.get_name() + "_uo")), var(f->generate_new_name(L.get_name() + "_ui")));
}
void block::unroll(var L, int fac, var o, var i) { FORALL(unroll(L, fac, o, i)); }
void block::vectorize(var L, int v) {
    function *f = children[0]->get_function();
    vectorize(L, v, var(f->generate_new_name(L.get_name() + "_vo")), var(f->generate_new_name(L.get_name() + "_vi")));
}
void block::vectorize(var L, int v, var o, var i) { FORALL(vectorize(L, v, o, i)); }
#undef FORALL

}  // namespace tiramisu
