/*
 * mgn_bench.h -- entry points of libmgn_hip that only test and benchmark harnesses use.
 *
 * None of them stands in for anything in the reference, and a host runtime that binds
 * mgn_hip.h does not need them: forcing a kernel family so that tests can drive every kernel
 * at every shape, and launch loops written in C for harnesses written in a scripting
 * language (an interpreter between launches would be what gets measured).
 */
#ifndef MGN_BENCH_H
#define MGN_BENCH_H

#include "mgn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Force a kernel family for the context's matmuls (default MGN_ROUTE_AUTO).  A family that
 * does not serve a shape makes the matmul return MGN_EINVAL ("... does not support this shape"). */
mgn_status mgn_ctx_set_route(mgn_ctx* ctx, mgn_route route);

/* How many times a wave polls for another workgroup's partial sums before it gives up (kernels whose
 * K parts meet without counters; default 2^20, far beyond any wait of a healthy launch).  With 0 a
 * reading wave looks at nothing and gives up at once, which is how a test makes that path run: the
 * kernels all end, the matmul's outputs are not valid and the next synchronising call returns
 * MGN_ETIMEOUT. */
mgn_status mgn_ctx_set_spin_limit(mgn_ctx* ctx, uint32_t polls);

/* The engine clock at this moment, as a kernel on the context's stream sees it (shader-clock ticks
 * against the constant 100 MHz counter over about 20 us); synchronises.  loaded = 0: one wave on an
 * otherwise idle device; loaded = 1: while every CU runs 16 waves of fp16 matrix instructions fed
 * from LDS, the mix of the several-row kernels.  Timings of instruction-bound kernels move with it
 * from box to box, bandwidth-bound ones do not.  cycles_per_round (may be null; 0 when not loaded):
 * shader cycles one wave of the load took per round of eight 4x4x4 fp16 matrix instructions and
 * four 16-byte LDS reads, with four such waves on its SIMD. */
mgn_status mgn_engine_clock_mhz(mgn_ctx* ctx, int loaded, float* mhz, float* cycles_per_round);

/* `steps` matmuls (mgn_matmul_q, or mgn_matmul_q_f16a when a_is_f16 != 0) enqueued back to back,
 * call i on weights[i % count]: the step loop of a compiled host
 * (examples/matmul_throughput.rs:114-127).  Copies of one weight in rotation keep it out of
 * the caches. */
mgn_status mgn_matmul_q_loop(mgn_ctx* ctx, const mgn_buf* a, int a_is_f16, const mgn_weight* const* weights,
                             size_t count, const mgn_buf* d, mgn_buf* c, uint32_t m, uint32_t steps);

/* `steps` launches, back to back like mgn_matmul_q_loop's, of a kernel that reads the packed
 * bytes of weights[i % count] (quants and scales) once and computes nothing.  Timed like a
 * matmul it gives the time the device needs for one launch plus one pass over a weight's
 * bytes: the floor a bandwidth-bound matmul on that weight can be held against.
 * pattern 0: every workgroup reads a contiguous share; pattern 1: the decode kernel's own map of
 * lanes to addresses (a wave per quad of columns, a lane per quant block, three blocks in flight),
 * which is the faster of the two on the weights that kernel is built for. */
mgn_status mgn_weight_read_loop(mgn_ctx* ctx, const mgn_weight* const* weights, size_t count, uint32_t steps, int pattern);

#ifdef __cplusplus
}
#endif
#endif /* MGN_BENCH_H */
