// A stand-in for the small part of Halide's run-time buffer API that Tiramisu wrapper programs
// use (the reference's tests/wrapper_test_*.cpp and benchmark wrappers include "Halide.h" only
// for Halide::Buffer<T>): a dense host array described by a halide_buffer_t with the pinned
// layout of generated code (benchmarks/linear_algebra/blas/level1/dot/generated_dot.o.h:1157-1219
// of the reference).  Dimensions are given and indexed innermost first, as in Halide:
// Buffer<float> A(K, M) is M rows of K contiguous elements and A(k, m) is element [m][k]
// ("indices are flipped", benchmarks/linear_algebra/blas/level3/sgemm/gpu/wrapper.cpp:59-62).
// Put this directory on the include path of a wrapper program instead of Halide's.
#ifndef TIRAMISU_AMD_HALIDE_SHIM_H
#define TIRAMISU_AMD_HALIDE_SHIM_H
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <string>
#include <vector>

#ifndef HALIDE_BUFFER_T_DEFINED
#define HALIDE_BUFFER_T_DEFINED
typedef struct halide_dimension_t { int32_t min, extent, stride; uint32_t flags; } halide_dimension_t;
typedef struct halide_type_t { uint8_t code, bits; uint16_t lanes; } halide_type_t;
typedef struct halide_buffer_t {
    uint64_t device;
    const void *device_interface;
    uint8_t *host;
    uint64_t flags;
    halide_type_t type;
    int32_t dimensions;
    halide_dimension_t *dim;
    void *padding;
} halide_buffer_t;
#endif

namespace Halide {

namespace shim {
template <class T> struct type_code { static constexpr uint8_t value = T(-1) < T(0) ? (T(1) / T(2) != T(0) ? 2 : 0) : 1; };
template <> struct type_code<bool> { static constexpr uint8_t value = 1; };
}  // namespace shim

template <class T>
class Buffer {
    struct storage {
        std::unique_ptr<T[]> owned;          // a plain array: Buffer<bool> must hand out bool *
        T *data = nullptr;                   // the array above, or memory of the caller's
        size_t count = 0;
        std::vector<halide_dimension_t> dims;
        halide_buffer_t raw;
        std::string name;
    };
    std::shared_ptr<storage> s;   // copies share the array, as Halide's do

    void build(const std::vector<int> &extents, T *existing = nullptr) {
        s = std::make_shared<storage>();
        size_t count = 1;
        s->dims.resize(extents.empty() ? 1 : extents.size());
        for (size_t d = 0; d < extents.size(); d++) {
            s->dims[d] = halide_dimension_t{0, extents[d], (int32_t)count, 0};
            count *= (size_t)extents[d];
        }
        s->count = count;
        if (!existing) s->owned.reset(new T[count > 0 ? count : 1]());
        s->data = existing ? existing : s->owned.get();
        std::memset(&s->raw, 0, sizeof(s->raw));
        s->raw.host = reinterpret_cast<uint8_t *>(s->data);
        s->raw.type = halide_type_t{shim::type_code<T>::value, (uint8_t)(8 * sizeof(T)), 1};
        s->raw.dimensions = (int32_t)extents.size();
        s->raw.dim = s->dims.data();
    }
    // indices beyond the buffer's dimensions are ignored, missing ones are 0
    template <class... I>
    size_t offset(I... idx) const {
        const int list[] = {(int)idx...};
        size_t o = 0;
        for (int d = 0; d < (int)sizeof...(I) && d < s->raw.dimensions; d++) o += (size_t)list[d] * (size_t)s->dims[d].stride;
        return o;
    }
    // extents followed, optionally, by a name (a label: print_buffer shows it)
    static void gather(std::vector<int> &, std::string &) {}
    static void gather(std::vector<int> &, std::string &name, const std::string &nm) { name = nm; }
    static void gather(std::vector<int> &, std::string &name, const char *nm) { name = nm; }
    template <class... R>
    static void gather(std::vector<int> &extents, std::string &name, int e, R... rest) {
        extents.push_back(e);
        gather(extents, name, rest...);
    }

public:
    Buffer() { build({}); }
    template <class... R>
    explicit Buffer(int e0, R... rest) {
        std::vector<int> extents;
        std::string nm;
        gather(extents, nm, e0, rest...);
        build(extents);
        s->name = nm;
    }
    explicit Buffer(const std::vector<int> &extents) { build(extents); }
    Buffer(const std::vector<int> &extents, const std::string &nm) { build(extents); s->name = nm; }
    // over memory that the caller owns
    Buffer(T *existing, const std::vector<int> &extents) { build(extents, existing); }
    Buffer(T *existing, const std::vector<int> &extents, const std::string &nm) { build(extents, existing); s->name = nm; }

    const std::string &name() const { return s->name; }
    halide_buffer_t *raw_buffer() { return &s->raw; }
    const halide_buffer_t *raw_buffer() const { return &s->raw; }
    // Generated functions of this build leave their results in host memory (explicit or
    // implicit copies), so the calls that wrappers make around Halide's GPU targets have nothing to do.
    int copy_to_host(void * = nullptr) { return 0; }
    int device_sync(void * = nullptr) { return 0; }
    void set_host_dirty(bool = true) {}
    void set_device_dirty(bool = true) {}
    T *data() { return s->data; }
    const T *data() const { return s->data; }
    T *begin() { return data(); }
    T *end() { return data() + s->count; }
    int dimensions() const { return s->raw.dimensions; }
    int extent(int d) const { return d < dimensions() ? s->dims[d].extent : 1; }
    int width() const { return extent(0); }
    int height() const { return extent(1); }
    int channels() const { return extent(2); }
    size_t number_of_elements() const { return s->count; }
    size_t size_in_bytes() const { return s->count * sizeof(T); }
    void fill(T v) { for (size_t i = 0; i < s->count; i++) s->data[i] = v; }
    void copy_from(const Buffer<T> &o) { for (size_t i = 0; i < s->count && i < o.s->count; i++) s->data[i] = o.s->data[i]; }

    // missing trailing indices are 0, so a 2-D buffer can be read as b(x, y, 0)
    template <class... I>
    T &operator()(int i0, I... rest) { return s->data[offset(i0, rest...)]; }
    template <class... I>
    const T &operator()(int i0, I... rest) const { return s->data[offset(i0, rest...)]; }
};

}  // namespace Halide
#endif
