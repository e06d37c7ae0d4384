// Internal to libsepcorr: shared between its translation units, not part of the C ABI.
#ifndef SEPCORR_INTERNAL_H
#define SEPCORR_INTERNAL_H
// Records `msg` as the calling thread's last error and returns `code`.
int sepcorr_set_error(int code, const char *msg);

// Fork/join on the library's two side streams per device, for calls whose kernels are independent of each other.
// sepcorr_fork makes *sa and *sb wait for everything queued on `user` and returns a token; when overlap is switched
// off (SEPCORR_SINGLE_STREAM=1, or per-kernel profiling) both are `user` itself.  sepcorr_join makes `user` wait for
// both and releases the token; it must be called on every path after a fork.  Capturable (events only).
void *sepcorr_fork(void *user, void **sa, void **sb);
int sepcorr_join(void *token);
#endif
