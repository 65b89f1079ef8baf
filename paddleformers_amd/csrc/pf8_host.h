// pf8_host.h -- host-side plumbing shared by the entry-point files: status codes, the thread-local
// error message and the launch check.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pf8.h"
#include "../../include/pf8_selftest.h"

// records the message for pf8_last_error() and returns `code`
int pf8_fail(int code, const char* where, const char* msg);
// hipGetLastError() -> PF8_OK or PF8_ELAUNCH (message recorded)
int pf8_check_launch(const char* where);
// compute units the GEMM grids may assume on the current device (pf8_set_num_cus, 0 = whole device)
int pf8_effective_cus();
// true when pf8_set_num_cus holds a budget below the current device's compute units
bool pf8_cus_capped();
// one line on stderr the first time note `id` (0..31) is raised in this process (PF8_QUIET=1 silences it): for launches
// that leave a kernel's fast path because of a size limit, which would otherwise only show as a slower call
void pf8_note_once(int id, const char* msg);
enum { PF8_NOTE_GROUPED_ORDER = 0, PF8_NOTE_MASKED_TABLE = 1 };

// Launches the 128x256 persistent forward kernel on a contiguous-grouped GEMM whose scales are UE8M0
// bytes (implemented next to that kernel; used by the UE8M0 entry point when a skewed expert load
// makes 256-row tiles wasteful).  pair_list: DEVICE work-item list of the paired-tile kernel; this kernel
// returns at once when that one takes the call (e8_paired_tiles_win).  cus: the compute-unit budget, read ONCE by
// the caller for both launches so that they reach the same decision.
int pf8_launch_deep_ue8m0(const uint8_t* p, const uint8_t* q, const uint8_t* sp8, const uint8_t* sq8, int64_t ldsq, void* out,
                          int64_t Prows, int64_t Qrows, int64_t red, int E, const int32_t* m_indices, const int32_t* pair_list,
                          int cus, hipStream_t stream, const char* where);

// Launches the 256x256-tile weight-gradient kernel (pf8_wgrad_e8.hip) on the listed experts of a grouped weight gradient
// whose scales are powers of two: item i is expert item_e[i], item_t0[i] 128-row blocks into the packed operands and
// item_kb[i] >= 4 blocks long; the list is ordered longest first.  Prows, Qrows: multiples of 128, at least 256.
constexpr int kWgE8MaxItems = 256;
int pf8_launch_wgrad_e8(const uint8_t* p, const uint8_t* q, const float* sp, const float* sq, float* out, int64_t Prows, int64_t Qrows,
                        int64_t ldo, int accumulate, int n_items, const int32_t* item_t0, const int32_t* item_kb, const uint8_t* item_e,
                        int cus, hipStream_t stream, const char* where);
// experts at least this many 128-row blocks long go to that kernel (0 = none); pf8_debug_set_wgrad_tile256_min_blocks
int pf8_wgrad_tile256_min_blocks();
