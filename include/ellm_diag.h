/*
 * ellm_diag.h — C ABI of libellm_diag.so, a measurement aid built beside the
 * attention library (not part of it, nothing in libellm_attn.so depends on it).
 * No counterpart in the reference.
 */
#ifndef ELLM_DIAG_H_
#define ELLM_DIAG_H_

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Enqueues one launch of a pure MFMA stream on `stream`: `workgroups` workgroups of four
 * waves (one per SIMD of a compute unit), each wave issuing iters x 32
 * v_mfma_f32_32x32x16 (dtype 0: f16, 1: bf16) on four independent accumulators with no
 * global memory access in the loop.
 *   mode 0: A and B operands stay in registers;
 *   mode 1: the A operand of every MFMA is re-read from LDS (ds_read_b128);
 *   mode 2: mode 1 plus the vector instructions a soft-max of the same tile shape costs
 *           (208 per 32 MFMAs, 32 of them exp2), dealt out between the MFMAs of the wave.
 * operands: device, [16][256] x 16 bytes (8 A and 8 B register images per lane,
 * interleaved), any 16-bit values of the chosen type — what the matrix pipe sustains
 * depends on them.  sink: device, workgroups x 256 floats.  *flops (may be NULL) receives
 * the floating-point operations of the launch.  Returns 0, 1 (bad argument) or 4 (launch
 * failed).
 */
int ellm_diag_mfma_stream(int mode, int dtype, const void* operands, float* sink, int workgroups,
                          int iters, void* stream, double* flops);

#ifdef __cplusplus
}
#endif
#endif /* ELLM_DIAG_H_ */
