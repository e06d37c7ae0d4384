// Internal to libsepcorr: shared between its translation units, not part of the C ABI.
#ifndef SEPCORR_INTERNAL_H
#define SEPCORR_INTERNAL_H
#include <stddef.h>
#include <stdint.h>
// Records `msg` as the calling thread's last error and returns `code`.
int sepcorr_set_error(int code, const char *msg);

// Fork/join on the library's two side streams per device, for calls whose kernels are independent of each other.
// sepcorr_fork makes *sa and *sb wait for everything queued on `user` and returns a token; when overlap is switched
// off (SEPCORR_SINGLE_STREAM=1, or per-kernel profiling) both are `user` itself.  sepcorr_join makes `user` wait for
// both and releases the token; it must be called on every path after a fork.  Capturable (events only).
void *sepcorr_fork(void *user, void **sa, void **sb);
int sepcorr_join(void *token);

// Per-kernel timing (sepcorr_profile_enable) for the other translation units: begin returns NULL while timing is off;
// end accepts NULL.  The label must be a string literal.
void *sepcorr_prof_begin(const char *name, void *stream);
void sepcorr_prof_end(void *token);

// Max/avg backward as gathers of feature rows (gather_backward.hip).  Eligible sizes only; `ws` holds
// sepcorr_gather_backward_bytes() bytes, 256-byte aligned.  d_f1 is enqueued on stream_f1, d_f2 on stream_f2 and the
// table of average gradients that d_f2 adds at its end on stream_table, which d_f2's last launch waits for through
// table_event (an event of the caller, recorded here; NULL keeps the table on stream_f2).  The three use disjoint
// parts of `ws`.
int sepcorr_gather_backward_eligible(int B, int H1, int W1, int H2, int W2, int C);
size_t sepcorr_gather_backward_bytes(int B, int H1, int W1, int H2, int W2, int C);
int sepcorr_gather_backward(const float *f1, const float *f2, const int32_t *am_u, const int32_t *am_v, const float *g_u,
                            const float *g_v, float *d_f1, float *d_f2, int B, int H1, int W1, int H2, int W2, int C, void *ws,
                            void *stream_f1, void *stream_f2, void *stream_table, void *table_event);
// table[b][v][c] = (1 / H2) sum_p g_v[p,1,v] f1[p,c] (gather_backward.hip), for the combined d_f2 kernel that leaves
// the average term of g_v to it.  Same sizes as the gather path; `part`: sepcorr_avg_table_v_part_bytes() of scratch.
int sepcorr_avg_table_v_eligible(int B, int H1, int W1, int H2, int W2, int C);
size_t sepcorr_avg_table_v_part_bytes(int B, int H1, int W1, int W2, int C);
int sepcorr_avg_table_v(const float *f1, const float *g_v, float *table, float *part, int B, int H1, int W1, int H2, int W2, int C,
                        void *stream);
#endif
