/*
 * Measurement aids of the fused LM-head library (same shared library as skyrl_lmhead.h).
 *
 * Nothing here stands in for an interface of the reference: these entry points exist for bench.py and the profiling
 * scripts -- the matrix pipe's own ceiling on a given kind of data, the device figures the published peak is made of, and
 * per-kernel HIP-event timing of the library's launches.  A trainer binding the path needs only skyrl_lmhead.h.
 */
#ifndef SKYRL_LMHEAD_BENCH_H
#define SKYRL_LMHEAD_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Measurement aid for benchmarks (no counterpart in the reference): what the matrix pipe sustains on a given kind of
 * data.  Launches `workgroups` workgroups of 4 wavefronts; each wavefront loads 32 operand fragments once from
 * `operands` (bf16, 32 fragments x 256 lanes x 8 values = 128 KiB) and then issues iters x 128 v_mfma_f32_16x16x32_bf16
 * in the order of the GEMM mainloop, with no memory access in the loop: 4 * workgroups * iters * 128 * 16384 flop.
 * `sink` receives 256 * workgroups floats.  On an MI355X the rate depends on the operand values (power): zeros run at the
 * published peak, N(0,1) operands well below it.
 */
int skyrl_lmhead_mfma_probe(const void* operands, int workgroups, int iters, float* sink, void* stream);

/*
 * Measurement aid (no counterpart in the reference): the fp32 atomic adds that a fully fused backward -- the variant
 * efficient_entropy_backward_kernel_general_mainloop_MN of fused_linear_logprob_triton.py:807-996, which this library does
 * not build -- would have to issue, and nothing else: one workgroup per 256 x 256 (vocab, token) tile adds 1.0 to its
 * [256, H] slice of d_weight (fp32 [V, H]) and of d_hidden (fp32 [T, H]); T and V multiples of 256.  Its duration is a lower
 * bound of that variant's, to set against the split backward's.  Both buffers are overwritten with counts.
 */
int skyrl_lmhead_atomic_floor_probe(float* d_weight, float* d_hidden, int64_t T, int64_t H, int64_t V, void* stream);

/* Measurement aid (no counterpart in the reference): compute units and maximum shader clock (kHz) of the current device, the
 * two figures the published matrix peak is made of (compute units x 4096 bf16 flop per clock x clock). */
int skyrl_lmhead_device_info(int* compute_units, int* max_clock_khz);

/*
 * Per-kernel timing for benchmarks (no counterpart in the reference, which times whole calls from Python with
 * torch.cuda.synchronize, skyrl/benchmarks/bench_fused_linear_logprob.py:96-101).
 * skyrl_lmhead_profile_begin() opens a profile on the calling thread and returns its handle (NULL if one is already open):
 * until it is closed, every kernel launched by skyrl_lmhead_fwd / skyrl_lmhead_bwd from this thread is bracketed by HIP
 * events on the launch stream.  skyrl_lmhead_profile_end() waits for those events, fills total_ms[k] and launches[k] for
 * k < skyrl_lmhead_num_kernel_kinds() and frees the profile.  skyrl_lmhead_kernel_name(k) names kind k.
 */
int skyrl_lmhead_num_kernel_kinds(void);
const char* skyrl_lmhead_kernel_name(int kind);
void* skyrl_lmhead_profile_begin(void);
int skyrl_lmhead_profile_end(void* handle, double* total_ms, int64_t* launches);

#ifdef __cplusplus
}
#endif
#endif /* SKYRL_LMHEAD_BENCH_H */
