/*
 * hexmi_calibrate.h - measurement probes exported by libhexmi.so. NOT part of
 * the operator ABI: nothing here stands in for an interface of the reference,
 * and an integrator binds include/hexmi.h only. bench.py uses these entry
 * points to put this GPU's own ceilings (what its matrix cores sustain on given
 * operand data, what vector work hides behind a matrix instruction, what an LDS
 * read pattern costs, what a compute unit takes in from L2) on record next to
 * the published peaks.
 *
 * Same conventions as hexmi.h (device pointers, stream as void*, int status).
 * Every launch is bounded: iters above HEXMI_CALIBRATE_MAX_ITERS (2^20, about a
 * minute of matrix instructions) is HEXMI_ETOOBIG.
 */
#ifndef HEXMI_CALIBRATE_H
#define HEXMI_CALIBRATE_H

#include "hexmi.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HEXMI_CALIBRATE_MAX_ITERS (1 << 20)

/* A stream of nothing but MFMAs (operands and accumulators in registers, no
 * memory traffic): what the matrix cores of this GPU sustain for one
 * instruction shape on operands of the caller's choice. It has no counterpart
 * in the reference; bench.py uses it to put the data-dependent, power-limited
 * ceiling of the MFMA-bound kernels on record next to the published peak.
 * shape: 0 = v_mfma_f32_32x32x16, 1 = v_mfma_f32_16x16x32; dtype HEXMI_F16 or
 * HEXMI_BF16; operands: 2 KiB, 16-byte aligned (lane l takes its A fragment at
 * byte 16*l and its B fragment at byte 1024 + 16*l, every wave the same);
 * waves_per_simd: 1 or 2; one workgroup per compute unit; sink: one float per
 * thread (hexmi_num_cus() * 256 * waves_per_simd), written once at the end.
 * shape 2 = v_mfma_f32_16x16x32 with the operand traffic of a GEMM tile: 8 x 8
 * accumulator tiles per wave, tile (i, j) fed by A fragment i and B fragment j
 * (operands: 16 KiB, A fragment i of lane l at byte 1024*i + 16*l, B fragment j
 * at byte 8192 + 1024*j + 16*l), one operand changing with every instruction;
 * waves_per_simd 1 only. The data-dependent rate is lower than with the same
 * two fragments throughout.
 * hexmi_mfma_peak_flops is the FLOP count of such a launch on this device. */
double hexmi_mfma_peak_flops(int shape, int waves_per_simd, int64_t iters);
int hexmi_mfma_peak(int shape, int dtype, const void *operands, int64_t iters,
                    int waves_per_simd, float *sink, hexmi_stream_t stream);

/* Two more measurement aids without a counterpart in the reference, both one
 * workgroup per compute unit, sink as above (hexmi_lds_read_pattern: 1024
 * floats per compute unit).
 *
 * hexmi_issue_slots: per MFMA of a registers-only stream (shape as above, fp16,
 * zero operands, 64 accumulator registers) per_mfma vector instructions of one
 * kind follow in the same wave: kind 0 = v_pk_add_f16, 1 = v_fma_f32,
 * 2 = v_exp_f32, 3 = v_fma_mix_f32 (one fp16 source), 4 = v_cvt_f32_f16;
 * per_mfma in {0,1,2,3,4,5,6,8}. The time per MFMA says how much
 * vector work a kernel can place between its MFMAs before the SIMD's
 * instruction issue, not the matrix pipe, sets the pace. The launch runs
 * iters * (4 for shape 0, 16 for shape 1) MFMAs per wave.
 *
 * hexmi_lds_read_pattern: 16 waves per compute unit issue only wave-wide
 * 16-byte LDS reads (iters * 8 per wave) with the lane-to-address pattern of
 * one of the tiled GEMM's fragment reads: 0 linear; 1 fp16 rows of 128 bytes
 * read as chunk 4*step + lane/16, swizzle (row>>1)&7; 2 the same rows read as
 * chunk 2*(lane/16) + step; 3 pattern 2 with the swizzle the int8-weight
 * kernel uses; 4 int8 rows of 64 bytes, swizzle (row>>2)&3; 5 the same with
 * (row>>1)&3 (in use); 6 pattern 1 unswizzled. */
int hexmi_issue_slots(int shape, int kind, int per_mfma, int64_t iters,
                      int waves_per_simd, float *sink, hexmi_stream_t stream);
int hexmi_lds_read_pattern(int pattern, int64_t iters, float *sink,
                           hexmi_stream_t stream);

/* hexmi_l2_stream: what a compute unit takes in from L2. One workgroup of 16
 * waves per compute unit streams `region_bytes` (a multiple of 64 KiB) `passes`
 * times in 1 KiB pieces per wave, to_lds != 0 straight into LDS
 * (global_load_lds, the path of the W8A16 kernels' copies), else into
 * registers; shared != 0: every workgroup reads the same region at the same
 * time, else workgroup b reads [b * region_bytes, (b + 1) * region_bytes) of
 * src, which must hold hexmi_num_cus() regions. Bytes moved:
 * hexmi_num_cus() * passes * region_bytes. sink: 1024 floats per compute unit.
 * passes * region_bytes above 64 GiB is HEXMI_ETOOBIG. */
int hexmi_l2_stream(int to_lds, int shared, int64_t region_bytes,
                    int64_t passes, const void *src, float *sink,
                    hexmi_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HEXMI_CALIBRATE_H */
