/*
 * CPU oracle for channels-last GroupNorm + fused activation, forward and backward.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithm of the reference's hot
 * path so that the HIP kernels can be checked against it.  Only tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py may build, load or call it; the shipped library never does.
 *
 * Reference functions restated (paths relative to the reference checkout):
 *   WelfordOps::reduce / project        src/gnnhwc/csrc/Welford.h:30-42, 66-72
 *   activations and derivatives         src/gnnhwc/csrc/gn_kernel.cu:62-106
 *   scale_shift_kernel (forward apply)  src/gnnhwc/csrc/gn_kernel.cu:350-409
 *   width_reduce / compute_dweight_dbias / compute_bwd_scale_biases / dx_elem_kernel
 *                                       src/gnnhwc/csrc/gn_kernel.cu:598-618, 717-727, 783-800, 868-871
 *   GN_Naive (closed form)              test/check_outputs.py:9-48
 *
 * The reference's CUDA sources cannot be compiled here (they need nvcc and the ATen headers), so there
 * is no oracle/_ref build.  What pins this restatement instead (tests/test_oracle.py):
 *   - torch.nn.functional.group_norm + the matching torch activation + autograd, in float64, on CPU:
 *     the library routine the reference's own tests compare against (test/check_outputs.py:91-157);
 *   - committed golden vectors made from that routine (tests/golden/);
 *   - brute-force Python loops for y and central finite differences of sum(dy * y) for dx, dgamma, dbeta
 *     on tiny inputs, including C = 1, G = C and G = 1;
 *   - invariants: sum(dx) = 0 over every (n, g) slab, mean 0 / variance var/(var+eps) of the normalised
 *     slab, invariance under a per-group shift and positive scaling of x.
 * Every exported function is covered by all of these; none is "parity unpinned".
 *
 * Two arithmetic widths are exported: *_f64 (the truth the GPU results are compared with) and *_f32
 * (float accumulation like the reference's T_ACC for float data, gn_kernel.cu:23-24; used as a CPU
 * timing leg).  Data layout: x, y, dy, dx are (N, R, C), C fastest; weight, bias (C); mean, rstd (N, G).
 */
#define _USE_MATH_DEFINES
#include <math.h>
#include <stdint.h>

#define REAL double
#define SUF f64
#include "gn_oracle_impl.h"
#undef REAL
#undef SUF

#define REAL float
#define SUF f32
#include "gn_oracle_impl.h"
#undef REAL
#undef SUF

int gn_oracle_version(void) { return 1; }
