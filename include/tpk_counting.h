/*
 * tpk_counting.h - the one extra entry point of libtpk_hip_counting.so.
 *
 * libtpk_hip_counting.so is libtpk_hip.so (same sources, same C ABI: tpk.h) with the distance
 * scans compiled -DTPK_COUNT_WORK: furthest point sampling, the ball queries, three_nn and the
 * Chamfer forward pass count the pair evaluations their lanes EXECUTE (one count = one lane
 * forming one squared distance; for furthest point sampling one running minimum updated).  It is
 * a measuring instrument for benchmarks - executed work divided by time, for kernels that skip
 * most of the pairs a brute-force scan would test - and slower than the shipping library (an
 * atomic add per lane at the end of every kernel).  It has no counterpart in the reference.
 */
#ifndef TPK_COUNTING_H
#define TPK_COUNTING_H

#ifdef __cplusplus
extern "C" {
#endif

/* Waits for the device, stores the pair evaluations counted on the current device since the last
 * call in *pairs and sets the counters back to zero.  Returns TPK_OK or a hipError_t. */
int tpk_work_read_reset(unsigned long long* pairs);

#ifdef __cplusplus
}
#endif
#endif /* TPK_COUNTING_H */
