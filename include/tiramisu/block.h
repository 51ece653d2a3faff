// A block groups computations so that one scheduling command is applied to all of them
// (reference: include/tiramisu/block.h, src/tiramisu_block.cpp:10-238).
#ifndef TIRAMISU_AMD_BLOCK_H
#define TIRAMISU_AMD_BLOCK_H
#include <vector>
#include <tiramisu/core.h>

namespace tiramisu {

class block : public computation {
    std::vector<computation *> children;
public:
    block(const std::vector<computation *> children);
    const std::vector<computation *> &get_children() const { return children; }

    void gpu_tile(var L0, var L1, int sizeX, int sizeY) override;
    void gpu_tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer,
                  var L0_inner, var L1_inner) override;
    void gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ) override;
    void gpu_tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer,
                  var L1_outer, var L2_outer, var L0_inner, var L1_inner, var L2_inner) override;
    void interchange(var L0, var L1) override;
    void interchange(int L0, int L1) override;
    void parallelize(var L) override;
    void shift(var L0, int n) override;
    void skew(var i, var j, int factor, var ni, var nj) override;
    void split(var L0, int sizeX) override;
    void split(var L0, int sizeX, var L0_outer, var L0_inner) override;
    void split(int L0, int sizeX) override;
    void tile(var L0, var L1, int sizeX, int sizeY) override;
    void tile(var L0, var L1, int sizeX, int sizeY, var L0_outer, var L1_outer, var L0_inner,
              var L1_inner) override;
    void tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ) override;
    void tile(var L0, var L1, var L2, int sizeX, int sizeY, int sizeZ, var L0_outer, var L1_outer,
              var L2_outer, var L0_inner, var L1_inner, var L2_inner) override;
    void tile(int L0, int L1, int sizeX, int sizeY) override;
    void tile(int L0, int L1, int L2, int sizeX, int sizeY, int sizeZ) override;
    void unroll(var L, int fac) override;
    void unroll(var L, int fac, var L_outer, var L_inner) override;
    void vectorize(var L, int v) override;
    void vectorize(var L, int v, var L_outer, var L_inner) override;
};

}  // namespace tiramisu
#endif
