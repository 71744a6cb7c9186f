/* PULP-NN layer API, 64-bit batch-norm parameters: link libpulpnn_hip64.so.
 * Mirrors /root/reference/64bit/include/pulp_nn_kernels.h. */
#ifndef PULP_NN_KERNELS_64_H
#define PULP_NN_KERNELS_64_H
#include <stdint.h>
#define PULP_NN_BN_T int64_t
#include "../pulp_nn_kernels_decl.h"
#endif
