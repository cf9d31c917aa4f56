// Host-side helpers shared by the translation units of libgalvatron_dp_hip.so (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/galvatron_dp_hip.h"

// Text of the calling thread's last error (what gdp_last_error() returns): a fixed thread-local buffer,
// so that reporting an error allocates nothing.
void gdp_clear_error();
int gdp_fail(int code, const char *msg);             // returns code
int gdp_fail_hip(hipError_t e, const char *what);    // GDP_E_NOMEM for an allocation failure, else GDP_E_HIP

// Host-side checks of one problem (instance number i is for the message only): sizes, null pointers,
// mem >= 1, other_mem >= 0, inter_index in range, no NaN / -inf, no possible overflow.  Allocates nothing.
int gdp_validate(const gdp_problem *p, int i);

// Index into GDP_VARIANTS of the register tile ts x r, or -1.
int gdp_find_variant(int ts, int r);
