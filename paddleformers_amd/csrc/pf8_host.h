// pf8_host.h -- host-side plumbing shared by the entry-point files: status codes, the thread-local
// error message and the launch check.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pf8.h"

// records the message for pf8_last_error() and returns `code`
int pf8_fail(int code, const char* where, const char* msg);
// hipGetLastError() -> PF8_OK or PF8_ELAUNCH (message recorded)
int pf8_check_launch(const char* where);
// compute units the GEMM grids may assume (pf8_set_num_cus, 0 = whole device)
int pf8_effective_cus();
