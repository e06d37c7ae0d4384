// Internal to libsepcorr: shared between its translation units, not part of the C ABI.
#ifndef SEPCORR_INTERNAL_H
#define SEPCORR_INTERNAL_H
// Records `msg` as the calling thread's last error and returns `code`.
int sepcorr_set_error(int code, const char *msg);
#endif
