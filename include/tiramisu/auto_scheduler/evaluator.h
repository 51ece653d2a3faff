#ifndef _TIRAMISU_AUTO_SCHEDULER_EVALUATOR_
#define _TIRAMISU_AUTO_SCHEDULER_EVALUATOR_

// Evaluation of candidates by execution: the part of the reference's auto-scheduler that the GPU path feeds
// (reference: include/tiramisu/auto_scheduler/evaluator.h:12-80, src/auto_scheduler/tiramisu_evaluator.cpp:14-125).
// The reference's candidates are syntax trees of loop transformations produced by its search (ast.h, which this
// build does not have); here a candidate carries options of the code-generation back-end -- tile shapes, steps
// fused per stencil launch, which emitter may take a nest -- set through function::set_backend_option.  The
// class keeps the reference's constructor and the signatures of evaluate() and get_measurements().

#include <map>
#include <string>
#include <vector>

#include <tiramisu/core.h>

namespace tiramisu::auto_scheduler
{

/**
  * A candidate to evaluate.  In the reference this is the auto-scheduler's abstract syntax tree with
  * the optimisations to apply; here it is the set of back-end options to generate code under.
  */
class syntax_tree
{
public:
    /** option name (function::set_backend_option) -> value */
    std::map<std::string, std::string> backend_options;

    syntax_tree() {}
    syntax_tree(std::map<std::string, std::string> const& options) : backend_options(options) {}

    /** "name=value name=value", or "default" for a candidate without options. */
    std::string to_string() const;
};

/**
  * An abstract class that represents an evaluation function (reference: evaluator.h:12-30).
  */
class evaluation_function
{
public:
    virtual ~evaluation_function() {}

    /** Takes a candidate and returns its evaluation (smaller is better). */
    virtual float evaluate(syntax_tree& ast) = 0;
};

/**
  * Evaluate programs by compiling and executing them (reference: evaluator.h:34-80).
  */
class evaluate_by_execution : public evaluation_function
{
protected:
    /** The program to compile and to execute. */
    tiramisu::function *fct;
    std::vector<tiramisu::buffer*> arguments;

    /** The name of the ".o" to generate (it will contain the compiled Tiramisu program); the shared
      * library made of it is obj_filename + ".so". */
    std::string obj_filename;

    /** The command that runs the wrapper: it loads the shared library, times the function and
      * prints one execution time per run on its standard output. */
    std::string wrapper_cmd;

    /** Generate code under the candidate's options and turn the object into a shared library. */
    void compile(syntax_tree& ast);

public:
    /** arguments : the input and output buffers of the program. */
    evaluate_by_execution(std::vector<tiramisu::buffer*> const& arguments,
                          std::string const& obj_filename,
                          std::string const& wrapper_cmd,
                          tiramisu::function *fct = tiramisu::global::get_implicit_function());

    /** Apply the candidate's options, compile the program and execute it; returns the first time the
      * wrapper prints (infinity when it prints none). */
    virtual float evaluate(syntax_tree& ast);

    /**
      * Apply the candidate's options, compile the program and execute it.
      * Returns the vector of measured execution times.
      * If the timeout parameter is defined, it stops the execution after MAX_RUNS*timeout seconds
      * (MAX_RUNS from the environment, 30 by default).
      * If exit_on_timeout is set to true, it raises an error when the timeout is reached and terminates the program.
      */
    std::vector<float> get_measurements(syntax_tree& ast, bool exit_on_timeout = false, float timeout = 0);
};

}

#endif
