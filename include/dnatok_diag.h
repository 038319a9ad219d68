/* Measurement aids of bench.py: libdnatok_diag.so, built from dnatok_amd/csrc/diag.hip.
 * Not part of the product library (libdnatok_hip.so, include/dnatok_hip.h) and not needed by any
 * caller of it: kernels that move memory in a given shape and do nothing else, so that an encoder's
 * rate can be set against what the machine gives that shape.  No counterpart in the reference. */
#ifndef DNATOK_DIAG_H
#define DNATOK_DIAG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 0 on success, a negative DNATOK_E_* code of include/dnatok_hip.h otherwise; the message of the
 * calling thread's last error in this library. */
const char *dnatok_last_error(void);

/* dst[0 .. bytes) = src[0 .. bytes): a workgroup copies contiguous 16 KB tiles (the fastest plain
 * copy measured on an MI355X).  Both buffers and the size are multiples of 16 bytes. */
int dnatok_diag_copy_tiles(const void *src, void *dst, size_t bytes, void *stream);

/* The loads and stores of dnatok_kmer_encode_padded's kernel for k = 6 on rows of plain bases,
 * without its arithmetic: rows read in steps of 1536 bytes (24 per lane), len / 6 ids and mask
 * bytes written per row (ids int32[n_rows, t_cap], mask uint8[n_rows, t_cap]; what is written
 * is not a tokenization), the cells up to fill_to as padding.  t_cap is a multiple of 4. */
int dnatok_diag_kmer_shape(const uint8_t *bytes, const int64_t *offsets, int64_t n_rows,
                           int64_t t_cap, int64_t fill_to, int32_t *ids, uint8_t *mask, void *stream);

/* libdnatok_hip_phases.so only (the whole product library compiled with -DDNATOK_BPE_PHASE_CYCLES;
 * same entry points as include/dnatok_hip.h, plus this one): where the teams of the BPE engine spent
 * their shader-clock cycles since the last reset, summed over all teams, as thread 0 of each team saw
 * them.  cycles[0..8] = initial pairs, round minimum, collect candidates, decide, late walks / scan,
 * apply, re-rank, refresh, output; cycles[12..15] = rounds, merges, positions, items (rows and chunks).
 * reset != 0 clears the cells afterwards.  Synchronises the device.  The instrumented kernels hold
 * more registers than the shipped ones: read the shares, not the totals. */
int dnatok_bpe_phase_cycles(unsigned long long *cycles, int reset);

#ifdef __cplusplus
}
#endif
#endif /* DNATOK_DIAG_H */
