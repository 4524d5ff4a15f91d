// Shared between the translation units of libftrocm.so; not part of the C-ABI.
#ifndef FTROCM_INTERNAL_H
#define FTROCM_INTERNAL_H

// Records a printf-style message for ftr_last_error() and returns 1.
int ftr_internal_fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// Device address of the static workspace on the current device; looked up
// once per device. Returns 0 on success. `ptr_out` may be NULL.
int ftr_internal_static_ws(void **ptr_out);

#endif
