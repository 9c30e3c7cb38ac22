/*
 * hip.h - internal face of the device shim (hip.c) and of the kernel launchers.
 * The exported C-ABI is include/darknet_hip.h; this header only adds what the library's own
 * translation units share.
 */
#ifndef DN_HIP_INTERNAL_H
#define DN_HIP_INTERNAL_H

#include "darknet_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Prints `msg` and ends the process, as the reference's error() does (src/utils.c:253-258). */
void dn_fatal(const char *msg);
/* Checks the sticky launch error after a kernel launch (check_error(cudaPeekAtLastError())
 * follows every launch in the reference, e.g. src/blas_kernels.cu:27). */
void dn_check_launch(const char *what);
/* Ends the process with a message naming `what` when the library is in parse-only mode
 * (hip_set_parse_only in darknet_hip.h). */
void hip_require_device(const char *what);
int hip_parse_only(void);
/* memcpy split over the host cores (a single core moves less than the host link does), and whether
 * [x, x+bytes) lies inside a buffer hip_host_alloc handed out */
void dn_host_copy(char *dst, const char *src, size_t bytes);
int dn_host_is_pinned(const void *x, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif
