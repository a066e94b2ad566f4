/*
 * Calibration aid of the benchmark, exported by libhiptk_calib.so (a separate library: nothing in
 * libhiptensor_amd.so calls or exports it).  No counterpart in the reference.
 */
#ifndef HIPTK_CALIB_H
#define HIPTK_CALIB_H

#ifdef __cplusplus
extern "C" {
#endif

/* The TFLOP/s a loop of nothing but the class's MFMA instruction (cls: a HIPTK_* class id of
 * hiptk_kernels.h) sustains on the current device (one 4-wave workgroup per CU), with constant
 * operands (random_operands = 0) or pseudo-random operands in [-1, 1) (1).  The clock the part
 * holds under a full matrix-core load depends on the operand data, so the second figure is the
 * practical ceiling for a contraction of random data.  Synchronous: loads the device for about
 * 150 ms first so that its clock has settled, then times 20 launches; allocates 4 KiB.
 * Returns 0 on success. */
int hiptk_mfma_ceiling(int cls, int random_operands, double* tflops);

#ifdef __cplusplus
}
#endif
#endif /* HIPTK_CALIB_H */
