// tiramisu::auto_scheduler::evaluate_by_execution for the HIP back-end
// (reference: src/auto_scheduler/tiramisu_evaluator.cpp:14-125).
#include <tiramisu/auto_scheduler/evaluator.h>

#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <iterator>
#include <limits>
#include <sstream>

namespace tiramisu::auto_scheduler
{

std::string syntax_tree::to_string() const
{
    std::string s;
    for (auto const& o : backend_options) s += (s.empty() ? "" : " ") + o.first + "=" + o.second;
    return s.empty() ? "default" : s;
}

evaluate_by_execution::evaluate_by_execution(std::vector<tiramisu::buffer*> const& arguments,
                                             std::string const& obj_filename,
                                             std::string const& wrapper_cmd,
                                             tiramisu::function *fct)
    : evaluation_function(), fct(fct), arguments(arguments), obj_filename(obj_filename), wrapper_cmd(wrapper_cmd)
{
    if (!fct) ERROR("evaluate_by_execution: no function (call tiramisu::init first)", true);
    fct->set_arguments(arguments);
}

// the directory this library was loaded from: the runtime library that generated objects link against lies beside it
static std::string library_directory()
{
    Dl_info info;
    if (!dladdr((void *)&library_directory, &info) || !info.dli_fname) return ".";
    std::string path = info.dli_fname;
    size_t slash = path.rfind('/');
    return slash == std::string::npos ? "." : path.substr(0, slash);
}

static std::string shell_quoted(std::string const& s)
{
    std::string r = "'";
    for (char c : s) { if (c == '\'') r += "'\\''"; else r += c; }
    return r + "'";
}

void evaluate_by_execution::compile(syntax_tree& ast)
{
    // Apply the candidate: its options replace the function's for this code generation
    const std::map<std::string, std::string> saved = fct->get_backend_options();
    for (auto const& o : ast.backend_options) fct->set_backend_option(o.first, o.second);

    // Compile the program to an object file (the whole pipeline: it can run again for the next candidate)
    fct->codegen(arguments, obj_filename, hardware_architecture_t::arch_amd_gpu);

    fct->clear_backend_options();
    for (auto const& o : saved) fct->set_backend_option(o.first, o.second);

    // Turn the object file to a shared library
    const std::string dir = library_directory();
    const std::string cmd = "g++ -shared -o " + shell_quoted(obj_filename + ".so") + " " + shell_quoted(obj_filename) +
                            " -L" + shell_quoted(dir) + " -ltiramisu_hip_wrappers -Wl,-rpath," + shell_quoted(dir);
    if (system(cmd.c_str()) != 0) ERROR("evaluate_by_execution: could not link " + obj_filename + ".so", true);
}

float evaluate_by_execution::evaluate(syntax_tree& ast)
{
    compile(ast);

    // Execute the wrapper and get execution time
    double exec_time = std::numeric_limits<double>::infinity();
    FILE *pipe = popen(wrapper_cmd.c_str(), "r");
    if (!pipe) return (float)exec_time;
    if (fscanf(pipe, "%lf", &exec_time) != 1) exec_time = std::numeric_limits<double>::infinity();
    // let the wrapper finish printing
    char buf[256];
    while (fgets(buf, sizeof buf, pipe)) {}
    pclose(pipe);
    return (float)exec_time;
}

std::vector<float> evaluate_by_execution::get_measurements(syntax_tree& ast, bool exit_on_timeout, float timeout)
{
    compile(ast);

    // define the execution command of the wrapper
    std::string cmd = wrapper_cmd;
    int nb_exec = 30; // by default
    if (std::getenv("MAX_RUNS") != NULL) nb_exec = std::atoi(std::getenv("MAX_RUNS"));
    if (timeout != 0) // the timeout for the total number of executions
        cmd = std::string("timeout ") + std::to_string(timeout * nb_exec) + std::string(" ") + wrapper_cmd;

    // execute the command and read its output
    FILE *pipe = popen(cmd.c_str(), "r");
    std::string output;
    if (pipe) {
        char buf[256];
        while (fgets(buf, sizeof buf, pipe)) output += buf;
    }
    const int status = pipe ? pclose(pipe) : -1;
    const int return_code = status >= 0 ? status / 256 : -1;
    if (exit_on_timeout && timeout != 0 && return_code == 124) {
        std::cerr << "error: Execution time exceeded the defined timeout " << timeout << "s * " << nb_exec << " executions" << std::endl;
        exit(1);
    }

    // parse the output into a vector of floats
    std::vector<float> measurements;
    std::istringstream iss(output);
    std::copy(std::istream_iterator<float>(iss), std::istream_iterator<float>(), std::back_inserter(measurements));
    if (measurements.empty()) {
        // no output: the execution failed, or no run finished before the timeout (then every run took at least that long)
        if (return_code == 124 && timeout != 0) measurements.push_back(timeout * 1000.f);
        else measurements.push_back(std::numeric_limits<float>::infinity());
    }
    return measurements;
}

}
