/* mi355_sage_test.h — switches of libmi355_sage.so that exist for its own tests and measurements.
 * Not part of the interface a caller binds (include/mi355_sage.h); process-wide, not thread-safe
 * against calls in flight. */
#ifndef MI355_SAGE_TEST_H
#define MI355_SAGE_TEST_H

#ifdef __cplusplus
extern "C" {
#endif

/* Attention scheduling.  mode 0: by shape and device (default); -1: never split; n > 0 (multiple
 * of 8, <= 1024): always split over n workgroups (fp16 variant, head dim up to 128; hand-over slots
 * a caller's workspace does not hold come from a library-owned per-stream buffer).  Returns 0, or -1
 * for a mode outside these. */
int mi355_sage_set_attn_split(int mode);

/* How long a workgroup of the split schedule polls for another workgroup's partial result before
 * it gives up, writes NaN into its rows and counts a fault.  polls > 0: that many polls of about a
 * microsecond (default 262144; the longest wait that can legitimately occur is one row tile's worth
 * of work, a few milliseconds); 0: back to the default; polls < 0: no workgroup announces its
 * result and every waiting one gives up after -polls polls, which is how the give-up path is
 * exercised without a hang. */
int mi355_sage_set_attn_split_wait(int polls);

/* Workgroups the split schedule would use for this shape on a device that supports it (256), or 0
 * for one workgroup per row tile: the rule alone, whatever the switch above and the device say. */
int mi355_sage_attn_split_rule(int B, int H, int N_q, int N_kv, int D, int variant);

#ifdef __cplusplus
}
#endif
#endif
