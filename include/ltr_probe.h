/*
 * ltr_probe.h - C ABI of libltr_probe.so: measurement helpers for benchmarks of the MI355X (gfx950) attention
 * library.  They are NOT part of the attention path and the product library (libltr_attn.so, ltr_attn.h) does not
 * contain them.  No counterpart in the reference: its only performance output is a printed wall time
 * (parallel/communication/ring_attention.py:195-196).  A benchmark prints the kernels' rates beside what the device
 * itself sustains.
 *
 * ltr_device_info - facts of the CURRENT device as hipDeviceProp reports them (host call, nothing is enqueued).
 *
 * ltr_probe_mfma - enqueues one kernel in which every wave of every CU (one block of 8 waves per CU) runs
 * 4 * iters v_mfma_f32_32x32x16_bf16 on register-resident operands: the device's matrix-pipe ceiling.
 * random_operands != 0: the operands are read once from workspace bytes [8192, workspace_bytes), which the caller
 * fills (random bf16 data makes the chip run at the clock its power limit allows); 0: constant operands.
 * Results, valid once the stream has finished: ((int64_t *)workspace)[0] = ticks of the constant 100 MHz wall clock
 * that ONE wave's loop took, [1] = ticks of the shader clock counter over the same interval: their ratio is the shader
 * clock under this load.  (The two waves of a SIMD do not alternate - the older one runs its loop at the pipe's full rate,
 * then the other - so the rate is taken over the launch's duration, timed by the caller with events on the stream:
 * CUs * 8 * iters * 4 * 32768 flop / seconds.)
 * workspace: device memory, 16-byte aligned, at least LTR_PROBE_MIN_WORKSPACE bytes.
 * Return value: 0 on success, a negative LTR_PROBE_E* code otherwise.
 */
#ifndef LTR_PROBE_H
#define LTR_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LTR_PROBE_OK 0
#define LTR_PROBE_EINVAL (-1)
#define LTR_PROBE_EALIGN (-3)
#define LTR_PROBE_ELAUNCH (-4)
#define LTR_PROBE_EDEVICE (-5)

typedef struct ltr_device_info_t {
    int32_t compute_units;
    int32_t clock_khz;            /* hipDeviceProp.clockRate: the engine clock the device advertises */
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int64_t lds_bytes_per_block;
    int64_t hbm_bytes;
    char arch[64];
} ltr_device_info_t;

#define LTR_PROBE_MIN_WORKSPACE (8192 + 65536)

int ltr_device_info(ltr_device_info_t *out);
int ltr_probe_mfma(void *workspace, int64_t workspace_bytes, int32_t iters, int32_t random_operands, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LTR_PROBE_H */
