// Helpers of Tiramisu wrapper programs (the functions the reference declares in
// include/tiramisu/utils.h:14-270 and its wrappers call): buffer initialisation, copy and
// comparison, timing.  They work on any Halide::Buffer<T> -- Halide's own or the stand-in of
// tiramisu/shim/Halide.h -- and do not need the compiler library.
#ifndef TIRAMISU_AMD_UTILS_H
#define TIRAMISU_AMD_UTILS_H
#include "Halide.h"      // Halide's own, or tiramisu/shim/Halide.h when that directory is on the include path (reference: utils.h:4)
#include <tiramisu/debug.h>
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

/** Set every element (reference: utils.h:23-35). */
template <typename T>
inline void init_buffer(Halide::Buffer<T> &buf, T val)
{
    for (int z = 0; z < buf.channels(); z++)
        for (int y = 0; y < buf.height(); y++)
            for (int x = 0; x < buf.width(); x++) buf(x, y, z) = val;
}

/** Element-wise copy of buffers of the same shape (reference: utils.h:68-88). */
template <typename T>
inline void copy_buffer(const Halide::Buffer<T> &from, Halide::Buffer<T> &to)
{
    if (from.dimensions() != to.dimensions() || from.channels() != to.channels() || from.height() != to.height() ||
        from.width() != to.width()) {
        std::cerr << "copy_buffer: the two buffers have different shapes" << std::endl;
        std::exit(1);
    }
    for (int z = 0; z < from.channels(); z++)
        for (int y = 0; y < from.height(); y++)
            for (int x = 0; x < from.width(); x++) to(x, y, z) = from(x, y, z);
}

/** Report a test's outcome; a failure is reported, not fatal (reference: utils.h:227-233). */
/** Prints the elements of a buffer of up to three dimensions, one row per line
  * (reference: utils.h:37-66). */
template <typename T>
inline void print_buffer(const Halide::Buffer<T> &buf)
{
    std::cout << "Printing " << buf.name() << "[";
    if (buf.channels() > 1) std::cout << buf.channels() << ",";
    if (buf.height() > 1) std::cout << buf.height() << ",";
    std::cout << buf.width() << "]: " << std::endl;
    for (int z = 0; z < buf.channels(); z++) {
        for (int y = 0; y < buf.height(); y++) {
            for (int x = 0; x < buf.width(); x++) {
                if (sizeof(T) == 1) std::cout << (int)buf(x, y, z);
                else std::cout << buf(x, y, z);
                if (x + 1 != buf.width()) std::cout << ", ";
            }
            std::cout << "\n";
        }
        std::cout << std::endl;
    }
    std::cout << std::endl;
}

inline void print_test_results(const std::string &test, bool success)
{
    if (success) std::cout << "\033[1;32mTest " << test << " succeeded.\033[0m" << std::endl;
    else std::cerr << "\033[1;31mTest " << test << " failed.\033[0m" << std::endl;
}

/** Exact comparison; the first mismatch is printed and ends the program with status 1
  * (reference: utils.h:155-180). */
template <typename T>
inline void compare_buffers(const std::string &test, const Halide::Buffer<T> &result, const Halide::Buffer<T> &expected)
{
    for (int z = 0; z < result.channels(); z++)
        for (int y = 0; y < result.height(); y++)
            for (int x = 0; x < result.width(); x++)
                if (result(x, y, z) != expected(x, y, z)) {
                    std::cerr << "\033[1;31mTest " << test << " failed. At (" << x << ", " << y << ", " << z
                              << "), expected: " << +expected(x, y, z) << ", got: " << +result(x, y, z) << ".\033[0m" << std::endl;
                    std::exit(1);
                }
    print_test_results(test, true);
}

/** One-sided comparison as the reference defines it: fails where result - expected exceeds the
  * threshold; the failure is reported and the function returns (reference: utils.h:91-123). */
template <typename T>
inline void compare_buffers_approximately(const std::string &test, const Halide::Buffer<T> &result,
                                          const Halide::Buffer<T> &expected, float threshold = 0.1f)
{
    if (result.dimensions() != expected.dimensions() || result.channels() != expected.channels() ||
        result.height() != expected.height() || result.width() != expected.width()) {
        std::cerr << "result has different dimension size from expected" << std::endl;
        std::exit(1);
    }
    for (int z = 0; z < result.channels(); z++)
        for (int y = 0; y < result.height(); y++)
            for (int x = 0; x < result.width(); x++)
                if ((float)(result(x, y, z) - expected(x, y, z)) > threshold) {
                    std::cerr << "\033[1;31mTest " << test << " failed. At (" << x << ", " << y << ", " << z
                              << "), expected: " << +expected(x, y, z) << ", got: " << +result(x, y, z) << ".\033[0m" << std::endl;
                    return;
                }
    print_test_results(test, true);
}

/** Median of a list of durations (reference: utils.cpp median()). */
inline double median(std::vector<std::chrono::duration<double, std::milli>> scores)
{
    if (scores.empty()) return 0.0;
    std::sort(scores.begin(), scores.end());
    const size_t n = scores.size();
    return n % 2 ? scores[n / 2].count() : (scores[n / 2 - 1].count() + scores[n / 2].count()) / 2.0;
}

/** Print the median time of each kernel (reference: utils.h:14-16). */
inline void print_time(const std::string &file_name, const std::string &kernel_name,
                       const std::vector<std::string> &header_text, const std::vector<double> &time_vector)
{
    std::cout << file_name << ": " << kernel_name << std::endl;
    for (size_t i = 0; i < header_text.size() && i < time_vector.size(); i++)
        std::cout << "    " << header_text[i] << ": " << time_vector[i] << " ms" << std::endl;
}
#endif
