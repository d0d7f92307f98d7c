/* Roofline.h — timing and roofline reporting for drivers of the operator entry points.
 *
 * Same header name and function names as the reference's helpers (t2s/src/Roofline.h:24-27,
 * Roofline.cpp:113-153), so that the LARGE branch of a driver written like
 * gemm-run-fpga.cpp:88-101 (compute_roof, number_ops, number_bytes, ExecTime(), roofline())
 * works against this library:
 *   ExecTime(name)   kernel time of the last operator call in ns.  The reference reads it from
 *                    <bitstream dir>/exec_time.txt (written by its OpenCL runtime,
 *                    AOT-OpenCL-Runtime.cpp:358-396); here it comes from t2sp_last_kernel_ns(),
 *                    or from the file named by $T2SP_EXEC_TIME_FILE when that is set (the entry
 *                    points write that file in the reference's format: first line the overall
 *                    ns, then one "<kernel_name> <ns>" line).
 *   roofline(...)    prints "GFlops: ..." like the reference and writes roofline.png (the file the
 *                    reference's drivers check for, gemm-run-fpga.cpp:101-104: both roofs and
 *                    the point, rasterised here instead of shelling out to matplotlib,
 *                    Roofline.py:24-56), plus roofline.svg (the same picture with its labels)
 *                    and roofline.txt (the numbers) into the current directory.  Units as in the reference:
 *                    mem_bandwidth in GB/s, compute_roof in MFLOP/s (it is divided by 1000 for
 *                    the plot, Roofline.py:33), number_ops in flop, exec_time in ns.
 *   DSPs(), FMax()   the reference multiplies 2*DSPs()*FMax() for the compute roof; here
 *                    DSPs() = fp32 MFMA multiply-add lanes of the device (CUs x 128) and
 *                    FMax() = its peak engine clock in MHz, so the same product is the fp32
 *                    matrix peak in MFLOP/s (256 CUs x 128 x 2 x 2400 MHz = 157.3 TFLOP/s).
 */
#ifndef T2SP_ROOFLINE_H
#define T2SP_ROOFLINE_H
#ifdef __cplusplus
int DSPs();
double FMax();
double ExecTime(const char *kernel_name = 0);
void roofline(double mem_bandwidth, double compute_roof, double number_ops, double number_bytes, double exec_time);
#endif
#endif
