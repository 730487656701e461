/* Measurement aids of the MI355X K-Quant packed-linear library's benchmark.
 *
 * Exported by libnfn_mi355_probes.so, a library of its own that only the
 * benchmark and the probes' test load: none of this is part of the path the
 * resident engine binds, and none of it has a counterpart in the reference.
 * Status codes as in nfn_mi355_tile_ops.h: 0 success, 1 argument violation,
 * anything else a HIP error code. */
#ifndef NFN_MI355_PROBES_H
#define NFN_MI355_PROBES_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int nfn_mi355_probes_abi_version(void);

/* Shader clock under load, a measurement aid (no counterpart in the reference;
 * for benchmarks that price a kernel against the matrix-core peak at the clock
 * the chip really ran at).  Enqueues one wave that waits about `microseconds`
 * (1..100000) on `cuda_stream` and then writes three uint64 to
 * `cycles_and_ticks` (device memory, 24 bytes): shader cycles, ticks of the
 * constant device clock, and that clock's ticks per second
 * (hipDeviceAttributeWallClockRate).  Launch it on a side stream while the work
 * under test runs on another. */
int nfn_mi355_shader_clock_probe_v1(
    uint64_t* cycles_and_ticks,
    int64_t microseconds,
    void* cuda_stream);

/* Matrix-core rates from registers, a measurement aid (no counterpart in the
 * reference): `groups` workgroups of four waves each run `steps` steps of one
 * 32 x 32 x 32 product per wave.  mode 0: fp16 operands (two
 * v_mfma_f32_32x32x16_f16); mode 1: int8 operands (one
 * v_mfma_i32_32x32x32_i8); mode 2: the int8 form a K-quant prefill with 16-bit
 * activation codes would need -- two int8 planes into fresh accumulators and,
 * after every 32 values, the rescale of all 16 accumulators by the sub-block's
 * scale; mode 3: one int8 plane (an 8-bit activation per 32-value group, the
 * reference's Q8_1 recipe) with the same rescale.  The benchmark times the
 * four and reports them side by side: the measurement behind the reserved
 * NFN_MI355_GEMM_INT8 mode.  `sink`: device
 * memory of one float per workgroup, never written in practice. */
int nfn_mi355_mfma_rate_probe_v1(int mode, int steps, int groups, float* sink, void* cuda_stream);

/* The floor under a launch, a measurement aid like the clock probe (no
 * counterpart in the reference): one workgroup per compute unit reads
 * `nbytes` of `data` (16-byte aligned; rounded down to whole 16-byte pieces per
 * workgroup) with plain coalesced loads and stores nothing; with nbytes = 0 it
 * is an empty kernel of the same grid.  Timed back to back in a graph over
 * the bytes a decode launch streams, it is what that launch would cost with
 * no arithmetic at all.  `sink`: device memory of one uint32 per compute unit
 * (1,024 bytes are enough), never written in practice. */
int nfn_mi355_read_probe_v1(
    const void* data,
    int64_t nbytes,
    uint32_t* sink,
    void* cuda_stream);

/* The read probe with `prefetch_rounds` x 512 16-byte pieces per workgroup of
 * `next` (the bytes the following launch will read, same size and split)
 * requested behind the first round of its own loads: measures whether a
 * launch can pull the next launch's first bytes into its XCD's L2 for free.
 * nbytes > 0; prefetch_rounds 0..64. */
int nfn_mi355_read_probe_chained_v1(
    const void* data,
    int64_t nbytes,
    const void* next,
    int prefetch_rounds,
    uint32_t* sink,
    void* cuda_stream);

#ifdef __cplusplus
}
#endif

#endif /* NFN_MI355_PROBES_H */
