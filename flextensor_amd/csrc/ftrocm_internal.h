// Shared between the translation units of libftrocm.so; not part of the C-ABI.
#ifndef FTROCM_INTERNAL_H
#define FTROCM_INTERNAL_H

// Records a printf-style message for ftr_last_error() and returns 1.
int ftr_internal_fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// The checks every launch descriptor has to pass before it is enqueued (module,
// argument array, grid and block extents). Returns 0 when the descriptor is fine.
struct ftr_launch_desc;
int ftr_internal_check_desc(const struct ftr_launch_desc *d);

// Device address of the static workspace on the current device; looked up
// once per device. Returns 0 on success. `ptr_out` may be NULL.
int ftr_internal_static_ws(void **ptr_out);

#endif
