/*
 * libfastlstm_hip.so -- diagnostics and test hooks.  Not part of the drop-in boundary (fastlstm_hip.h): nothing
 * here has a counterpart in the reference, a product caller needs none of it, and all of it is process-wide
 * state or measurement code.  Used by the tests (to put two kernel families side by side on the same inputs, to
 * force the time-out path from the host) and by bench.py (the step-latency probe, the clock traces).
 */
#ifndef FASTLSTM_HIP_DIAG_H
#define FASTLSTM_HIP_DIAG_H

#include "fastlstm_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Diagnostics: which kernel families the recurrent entry points may choose besides the general kernels: bit 0 =
 * the XCD-local kernels, bit 1 = the register-resident kernels of H = 1280 ... 2048, bit 2 = the form of their
 * reverse kernel in which teams of workgroups split the sums over K (default 7: all).  With 0
 * every shape runs the general kernels, which lets a test or a measurement put two families side by side on
 * the same inputs.  Process-wide; no counterpart in the reference. */
void fastlstm_set_kernel_families(int mask);
int fastlstm_get_kernel_families(void);

/* Measurement: with `on` != 0 the stand-alone 16-bit GEMM launches (fastlstm_gemm_ifgo, _dx, _wgrad) run the tile
 * kernel in its earlier form -- one tile per workgroup, symmetric main loop, C staged through LDS and written with
 * ordinary stores, the weight gradients as two products followed by a column-sum pass -- so that a benchmark can
 * time both forms on the same operands in one process (the results agree to rounding; bench.py reports both).
 * Process-wide, default 0; no counterpart in the reference. */
void fastlstm_set_gemm_baseline(int on);

/* Upper bound, in 100 MHz ticks, a barrier wait may spin before it gives up
 * (default 4e8 = 4 s).  Tests lower it to force the time-out path from the host. */
void fastlstm_set_spin_limit(long long ticks);

/* Diagnostics: when `buf` (device memory, 32 bytes per workgroup of the largest GEMM grid)
 * is non-NULL the 16-bit GEMM kernels record 4 stamps of the 100 MHz clock per workgroup
 * (start, main loop entered, main loop left, done).  NULL switches it off (default). */
void fastlstm_set_gemm_trace(void *buf);

/* Diagnostics: when `buf` (zero-filled device memory, 32 bytes per workgroup) is non-NULL the
 * recurrent kernels accumulate, per workgroup and in 100 MHz ticks, four phase times: forward =
 * waiting for peers, operand fetch + MFMA, reduce + gate maths, publish; backward = gate maths,
 * publish + stores, waiting for peers, operand fetch + MFMA + reduce. */
void fastlstm_set_recurrent_trace(void *buf);

/* Diagnostics: the latency bound of one recurrence step.  Runs `steps` rounds of the links of a timestep
 * that no arithmetic throughput removes, with the recurrent kernels' own barrier and exchange code:
 * mode 0 = the empty barrier (publish + wait), 1 = + every member stores its share of a `rows`-row fp16 h
 * tile into the step's exchange slot (slot t % 2), 2 = + every wave fetches its operand blocks of the step
 * (loads that go past the L1, as in the kernels); 3, 4 (kind 0 only) = the exchange without a barrier:
 * consumers poll the data itself, unwritten values hold an all-ones sentinel, loads bypass the L1 (sc1 /
 * sc0 sc1); the exchange slots of ws (everything from byte 66560 on) must then hold 0xFF bytes.
 * kind 0 = an XCD-local group of `members` <= 32 workgroups (counters in that XCD's L2), kind 1 = a flag
 * group of `members` <= 256 workgroups over all XCDs (device-scope flags).  H <= 2048, a multiple of 32 and of
 * `members`; rows = 16, 32, 48 or 64 batch rows per group.  The caller times the launch (its duration /
 * steps = microseconds per round); ws: zeroed device memory of fastlstm_diag_step_probe_bytes.  No
 * counterpart in the reference. */
int fastlstm_diag_step_probe(int kind, int mode, int members, int H, int rows, int steps, void *ws,
                             size_t ws_bytes, void *stream);
size_t fastlstm_diag_step_probe_bytes(int steps, int H, int rows);

#ifdef __cplusplus
}
#endif
#endif /* FASTLSTM_HIP_DIAG_H */
