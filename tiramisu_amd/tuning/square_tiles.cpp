// Checks the back-end's tile model against the machine: for every size n given on the command line (default
// 1024 2048 3072 4096) the n x n x n sgemm program is generated under each square tile of the MFMA kernel that
// divides n (back-end option "mfma_tile": 64, 128, 192, 256) and once with no option at all (what the back-end
// chooses by itself), every candidate is compiled, linked and timed on the GPU through
// tiramisu::auto_scheduler::evaluate_by_execution, and one JSON line per size says which tile the model of
// kernels/target_gfx950.h picks (ttarget::square_tile_for), which one ran fastest, and whether they agree.
//
//     square_tiles <scratch directory> [--wrapper "<command prefix>"] [n ...]
//
// The wrapper command (default: python3 -m tiramisu_amd.autotune --time) is run as
// "<prefix> <library> <function> <manifest>" and prints one time in milliseconds per run.
// Needs a GPU at run time; built on demand (tiramisu_amd/autotune.py: build_tuner), not with the programs.
#include <tiramisu/tiramisu.h>
#include <tiramisu/auto_scheduler/evaluator.h>

#include <algorithm>
#include <cstdlib>
#include <iostream>

#include "../csrc/kernels/target_gfx950.h"

using namespace tiramisu;

// the sgemm program of tiramisu_amd/programs/sgemm.cpp with its GPU schedule
static std::vector<buffer *> sgemm_program(int n, const std::string &name)
{
    tiramisu::init(name);
    var i("i", 0, n), j("j", 0, n), k("k", 0, n), s("s", 0, 2);
    buffer *b_scal = new buffer("b_scal", {2}, p_float32, a_input);
    buffer *b_A = new buffer("b_A", {n, n}, p_float32, a_input);
    buffer *b_B = new buffer("b_B", {n, n}, p_float32, a_input);
    buffer *b_C = new buffer("b_C", {n, n}, p_float32, a_output);
    input *scal = new input("scal", {s}, p_float32);
    scal->store_in(b_scal);
    constant *alpha = new constant("alpha", (*scal)(0));
    constant *beta = new constant("beta", (*scal)(1));
    input *A = new input("A", {i, k}, p_float32);
    input *B = new input("B", {k, j}, p_float32);
    A->store_in(b_A);
    B->store_in(b_B);
    computation *acc_init = new computation("acc_init", {i, j}, expr((float)0));
    computation *acc = new computation("acc", {i, j, k}, p_float32);
    acc->set_expression((*acc)(i, j, 0) + (*A)(i, k) * (*B)(k, j));
    computation *C = new computation("C", {i, j}, p_float32);
    C->set_expression((*acc)(i, j, 0) * (*alpha) + (*C)(i, j) * (*beta));
    C->store_in(b_C);
    b_A->tag_gpu_global();
    b_B->tag_gpu_global();
    b_C->tag_gpu_global();
    buffer *acc_reg = new buffer("acc_reg", {1}, p_float32, a_temporary);
    acc_reg->tag_gpu_register();
    computation *acc_decl = new computation("acc_decl", {i, j}, allocate(*acc_reg));
    acc_init->store_in(acc_reg, {0});
    acc->store_in(acc_reg, {0});
    var ib("ib"), jb("jb"), it("it"), jt("jt");
    block({acc_decl, acc_init, acc, C}).gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    acc_decl->then(*acc_init, jt).then(*acc, jt).then(*C, jt);
    return {b_scal, b_A, b_B, b_C};
}

static float median(std::vector<float> v)
{
    std::sort(v.begin(), v.end());
    return v.empty() ? 0.f : v[v.size() / 2];
}

int main(int argc, char **argv)
{
    if (argc < 2) {
        std::cerr << "usage: square_tiles <scratch directory> [--wrapper \"<command prefix>\"] [n ...]" << std::endl;
        return 2;
    }
    const std::string scratch = argv[1];
    std::string wrapper = "python3 -m tiramisu_amd.autotune --time";
    std::vector<int> sizes;
    for (int a = 2; a < argc; a++) {
        if (std::string(argv[a]) == "--wrapper" && a + 1 < argc) wrapper = argv[++a];
        else sizes.push_back(std::atoi(argv[a]));
    }
    if (sizes.empty()) sizes = {1024, 2048, 3072, 4096};
    int disagreements = 0;
    for (int n : sizes) {
        const std::string name = "sgemm_tiles_" + std::to_string(n);
        const std::vector<buffer *> arguments = sgemm_program(n, name);
        const std::string obj = scratch + "/" + name + ".o";
        auto_scheduler::evaluate_by_execution evaluator(arguments, obj, wrapper + " " + obj + ".so " + name + " " + obj + ".json");
        std::vector<std::pair<std::string, float>> times;
        auto_scheduler::syntax_tree chosen;                       // no option: the back-end's own choice
        times.push_back({"default", median(evaluator.get_measurements(chosen))});
        for (int tile : {64, 128, 192, 256}) {
            if (n % tile != 0) continue;
            auto_scheduler::syntax_tree candidate({{"mfma_tile", std::to_string(tile)}});
            times.push_back({std::to_string(tile), median(evaluator.get_measurements(candidate))});
        }
        const int model = ttarget::square_tile_for(n, n);
        std::string fastest;
        float best = 0;
        for (size_t c = 1; c < times.size(); c++)
            if (fastest.empty() || times[c].second < best) { fastest = times[c].first; best = times[c].second; }
        const bool agrees = fastest == std::to_string(model);
        disagreements += agrees ? 0 : 1;
        std::cout << "{\"size\": " << n << ", \"model_tile\": " << model << ", \"fastest_tile\": " << fastest << ", \"agrees\": " << (agrees ? "true" : "false")
                  << ", \"ms\": {";
        for (size_t c = 0; c < times.size(); c++) std::cout << (c ? ", " : "") << "\"" << times[c].first << "\": " << times[c].second;
        std::cout << "}}" << std::endl;
    }
    return 0;
}
