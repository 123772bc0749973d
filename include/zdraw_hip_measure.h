/*
 * zdraw_hip_measure.h: measurement aids of libzdraw_hip.so. NOT FOR CALLERS.
 *
 * Nothing here has a counterpart in the reference's bridge (src/metal/metal_c.zig) and a
 * renderer never calls any of it: the benchmark and the tests use these entries to choose
 * between builds of one kernel and to read the shader clock a launch really ran at. They
 * change process-wide state and are not part of the drop-in boundary (include/zdraw_hip.h).
 *
 * The library itself reads no environment variable for any of this.
 */
#ifndef ZDRAW_HIP_MEASURE_H
#define ZDRAW_HIP_MEASURE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Clock probe. While on, every workgroup of an attention launch records how long it ran in
 * shader-clock cycles and in ticks of the fixed 100 MHz reference counter; cycles / ticks x
 * 0.1 is the clock in GHz that the kernel really ran at (under load the power limit sets
 * it). clock_probe_read waits for the last probed launch and copies the first `capacity`
 * workgroups' figures (in launch order); it returns how many. */
void zdraw_hip_clock_probe(int on);
size_t zdraw_hip_clock_probe_read(uint64_t* cycles, uint64_t* ref_ticks, size_t capacity);

/* Which build of the attention kernel runs. Bit 0: 0 = 8 waves x 32 query rows per
 * workgroup, one workgroup per CU (default); 1 = 4 waves x 32 query rows, two workgroups
 * per CU. Bit 1: 2 = never split the tiles of a thinly filled last round along the keys
 * (by default they are). */
void zdraw_hip_set_attention_variant(int variant);

/* Which build multiplies 256 x 256 tiles of 16-bit activations. 1 = four waves, 128 x 128
 * each (default); 0 = eight waves, 64 x 128 each. */
void zdraw_hip_set_gemm_build(int build);

/* How many query tiles (128 rows) of the last wide-head launch had a score outgrow its row's
 * fixed reference point and were formed again by the running-maximum kernel (waits for that
 * launch). 0 on ordinary data; -1 if no wide-head launch has been made or the read failed. */
int zdraw_hip_wide_redo_tiles(void);

/* A queue as zdraw_hip_create_queue makes it, its stream confined to cu_count compute units
 * (0 < cu_count < the device's CU count; anything else: an ordinary queue): does a kernel's
 * time follow the CU count or the board's power limit. */
void* zdraw_hip_create_queue_on_cus(void* device, int cu_count);

#ifdef __cplusplus
}
#endif
#endif
