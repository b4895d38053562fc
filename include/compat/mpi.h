/* Minimal stand-in used only when no MPI installation provides <mpi.h>.
 * The API takes an MPI_Comm for source compatibility with ROC_SHMEM
 * (library/include/roc_shmem.hpp:144,157 in the reference); nothing in this
 * library communicates through MPI. */
#ifndef ROCSHMEM_MI355X_COMPAT_MPI_H
#define ROCSHMEM_MI355X_COMPAT_MPI_H

typedef int MPI_Comm;
#ifndef MPI_COMM_WORLD
#define MPI_COMM_WORLD ((MPI_Comm)0x44000000)
#endif

#endif
