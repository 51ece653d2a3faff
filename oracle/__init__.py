"""Parity oracle: TEST INFRASTRUCTURE, not part of the product.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import or run anything
in this package.  It holds CPU restatements of what the reference computes on the hot path:

* reference_loops.py  numpy restatements of the nested-loop references that the reference's own
                      wrapper programs compare against (tests/wrapper_test_*.cpp) and of the
                      five benchmark computations;
* cpu_backend/        a restatement of the reference's CPU back-end (loop tags -> C + OpenMP
                      from the same isl AST), used to compile the CPU-scheduled variant of each
                      Tiramisu program: the "reference's own CPU-generated code" of the parity
                      statement, and the timed CPU baseline.

Parity status per function is listed at the top of each file.
"""
