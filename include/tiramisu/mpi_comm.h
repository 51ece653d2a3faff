// Programs of the reference include this header whether or not they are built with MPI
// (reference: include/tiramisu/mpi_comm.h, whose declarations all sit under WITH_MPI).  This build is for
// one GPU in one process and has no MPI layer: the header exists so that those programs compile.
#ifndef TIRAMISU_AMD_MPI_COMM_H
#define TIRAMISU_AMD_MPI_COMM_H
#ifdef WITH_MPI
#error "this build of Tiramisu has no MPI layer: compile without WITH_MPI"
#endif
#endif
