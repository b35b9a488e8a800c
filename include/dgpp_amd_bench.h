/* Measurement aids of libdgpp_amd.so: A/B switches and streaming probes used by the benchmark and by the tests that
 * compare kernel forms. Nothing here is part of the drop-in launcher surface (dgpp_amd.h does not include this
 * file) and no product caller needs it. */
#ifndef DGPP_AMD_BENCH_H
#define DGPP_AMD_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Bench A/B switches, process-wide relaxed atomics (a set that races a launch is defined: the launch takes the old or
 * the new value), 0 everywhere = the product behaviour. They are inert unless the process opted in through the
 * environment (DGPP_AMD_BENCH=1, see dgpp_tune_enabled); a library built with -DDGPP_NO_TUNE leaves them out
 * (dgpp_tune_set stores nothing, dgpp_tune_get returns 0). The reference keeps such a switch in its launcher header
 * too: moe_set_fp8_ldm, src/kernels/glm_moe_launch.hpp:90.
 * key 0: preferred chunks per lane of the row geometry (0 = default 4); key 1: slots of one expert a
 * decode-slot block serves together (0 = default: 2 gate/up, 4 down; 1 = one slot per block);
 * key 2: row steps per block of the slot launches (0 = automatic); key 3: 1 stages activations before
 * any weight load is issued (default: activation loads, first weight pass, LDS commit); key 4: 1 keeps
 * the layer driver on the two-launch down + accumulate form; key 5: 2 moves every GEMV launcher to the
 * matrix-core form, 1 keeps the dense launchers on the vector core at every row count (default: the dense launchers
 * choose by rows, matrix size and workspace); key 6: 1 makes the layer driver compute the slot order for small decode batches too
 * (default: batches of at most 128 routed slots find the sharers of an expert by ballot, no order);
 * key 7: 1 keeps the selection of a one-token step a launch of its own (default: repeated in the gate/up
 * blocks, dgpp_launch_moe_select_gate_up_swiglu); key 8: row tiles an XCD takes for one token before it turns to the next token in the token-major
 * down + accumulate launch (0 = automatic: 1 from 64 routed slots on, else plain token-major order);
 * key 9: 1 keeps the shared expert's passes of the layer driver
 * on the caller's stream, 2 moves them to a second stream beside the routed passes at every batch size (default:
 * from three tokens on); 3 and 4 keep one stream and never / always fold the accumulation into the shared down pass
 * (default: at one token); key 10: 2 or 4 runs the router's token-tiled score kernel at every batch size with that many tokens per
 * wavefront (0 = automatic: tiled from 32 rows on, 4 tokens from 128 rows on); key 11: the dense matrix-core launch
 * without a workspace that runs the four parts of K side by side inside a block: 1 never, 2 always with four row groups
 * per block, 3 with two for up to eight rows (0 = automatic: four while the row tiles fit one round of the chip, two for up
 * to a round and a quarter); key 12: 1 makes dgpp_launch_moe_slot_chain* run the launches the one-launch chain stands for, 2 makes
 * the layer driver take the one-launch chain for small routed-only decode batches (default: the driver runs the
 * launches; the chain measured slower); key 13: row steps per wavefront of the chain's down part (0 = automatic);
 * key 14: the fused gate + up matrix-core grouped launch: 1 = every wavefront walks both matrices in turn, 2 = the block's
 * wavefronts split into gate walkers and up walkers (0 = automatic: split while the grid is at most 2048 blocks). Outputs do not
 * depend on keys 1 - 4 and 6 - 14; keys 0 and
 * 5 change the fp32 summation order (every GEMV launcher follows them alike, so the launchers stay
 * bitwise twins of each other). */
void dgpp_tune_set(int key, int value);
int dgpp_tune_get(int key);
/* 1 when the process opted in: the switches take values only if the environment held DGPP_AMD_BENCH=1 at the first
 * call of dgpp_tune_set / dgpp_tune_enabled (read once). Without it dgpp_tune_set stores nothing and every launcher
 * runs its measured default, whatever any component of the process calls. */
int dgpp_tune_enabled(void);

/* Measurement aid with no counterpart in the reference: a plain streaming copy of `bytes`
 * (a multiple of 16; both pointers 16-byte aligned) on `stream`. A profiler's HBM byte counters
 * are calibrated against it: it reads `bytes` and writes `bytes`, nothing else. */
int dgpp_probe_copy(void* dst, const void* src, size_t bytes, void* stream);

/* A plain streaming READ of `bytes` (a multiple of 16, 16-byte aligned) on `stream`: 16-byte loads, eight in flight
 * per lane, nothing stored (`sink`, at least 8192 words, is written only for a checksum no input produces). `blocks`
 * blocks of 256 threads (0 = 2048, at most 8192); span != 0 gives every block one contiguous span of the buffer, span == 0
 * lets the whole grid stride through it together. The rate it reaches is the ceiling of a weight stream on this chip;
 * nontemporal != 0 uses the nontemporal load form the GEMV kernels use where a launch reads its weights once. */
int dgpp_probe_read(const void* src, size_t bytes, void* sink, int nontemporal, int blocks, int span, void* stream);

#ifdef __cplusplus
}
#endif
#endif
