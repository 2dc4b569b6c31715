// Shared by the HIP sources of libparalia.so, not part of the exported interface: both record the text that
// pl_last_error() returns on the calling thread and hand back the status code to return.
#ifndef PARALIA_PL_INTERNAL_H
#define PARALIA_PL_INTERNAL_H

int pl_fail_hip(int hip_error, const char* what);   // "<what>: <HIP error string>", returns PL_ERR_HIP
int pl_fail_msg(int code, const char* message);     // returns code

// Resolves, once per device, the address of the fixed scratch array behind pl_dgemv_noalloc on the current device.
int pl_noalloc_setup_current_device(void);

#endif
