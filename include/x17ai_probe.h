/* x17ai_probe.h -- measurement aids of the benchmark.  NOT part of the drop-in boundary and without any counterpart
 * in the reference: three small kernels whose only purpose is to calibrate what the benchmark reports against the
 * machine at hand.  They live in their own library (libx17ai_probe.so), built on the operator layer of
 * include/x17ai_host.h, whose device and tensor handles they take.
 *
 * Every function returns 0 on success; on failure x17p_last_error() holds the message. */
#ifndef X17AI_PROBE_H
#define X17AI_PROBE_H

#include <stddef.h>
#include "x17ai_host.h"

#ifdef __cplusplus
extern "C" {
#endif

char const *x17p_last_error(void);

/* A plain device-to-device copy kernel of known size, against which HBM-traffic counters are calibrated
 * (src and dst: equal sizes, a multiple of 16 bytes). */
typedef struct X17pCopyProbe X17pCopyProbe;
int x17p_copy_probe_new(X17hDevice *dev, X17pCopyProbe **out);
void x17p_copy_probe_free(X17pCopyProbe *p);
int x17p_copy_probe_launch(X17pCopyProbe *p, X17hTensor *src, X17hTensor *dst);

/* A loop of nothing but matrix-core instructions on register operands taken from `operands` (at least 98304 bytes;
 * what the machine sustains depends on their values).  kind: 0 int8, 1 e4m3, 2 f16.  `out` takes 4 bytes per
 * thread (256 x 512); *ops receives the operations launched. */
typedef struct X17pMfmaProbe X17pMfmaProbe;
int x17p_mfma_probe_new(X17hDevice *dev, int kind, X17pMfmaProbe **out);
void x17p_mfma_probe_free(X17pMfmaProbe *p);
int x17p_mfma_probe_launch(X17pMfmaProbe *p, X17hTensor *operands, X17hTensor *out, size_t iterations, double *ops);

/* A loop of one vector (or scalar) instruction on sixteen independent registers, one wavefront per workgroup,
 * 1024 * waves_per_simd workgroups.  op: index into the table of probes/valu_probe.hip (x17p_valu_probe_op_name).
 * `src` holds at least 80 floats, `out` 4 bytes per thread launched; *instructions receives the number of
 * wavefront-instructions each SIMD executes (waves_per_simd * iterations * 16). */
typedef struct X17pValuProbe X17pValuProbe;
int x17p_valu_probe_ops(void);
char const *x17p_valu_probe_op_name(int op);
int x17p_valu_probe_new(X17hDevice *dev, int op, X17pValuProbe **out);
void x17p_valu_probe_free(X17pValuProbe *p);
int x17p_valu_probe_launch(X17pValuProbe *p, X17hTensor *src, X17hTensor *out, size_t waves_per_simd, size_t iterations,
                           double *instructions);

#ifdef __cplusplus
}
#endif
#endif /* X17AI_PROBE_H */
