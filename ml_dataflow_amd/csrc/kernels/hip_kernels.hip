/*
 * hip_kernels.hip -- the single translation unit that becomes hip_kernels_gfx950.hsaco, the code object
 * the handle loads with hipModuleLoad (the counterpart of the reference's cuda_kernels.cu -> .cubin).
 */
#include "routing.hip"
#include "movement.hip"
#include "norm.hip"
#include "optimizer.hip"
#include "cast.hip"
