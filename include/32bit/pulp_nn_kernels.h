/* PULP-NN layer API, 32-bit batch-norm parameters: link libpulpnn_hip32.so.
 * Mirrors /root/reference/32bit/include/pulp_nn_kernels.h. */
#ifndef PULP_NN_KERNELS_32_H
#define PULP_NN_KERNELS_32_H
#include <stdint.h>
#define PULP_NN_BN_T int32_t
#include "../pulp_nn_kernels_decl.h"
#endif
