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
// mem >= 0, other_mem >= 0, inter_index in range, no NaN / -inf, no possible overflow -- everything but the
// initial costs.  Allocates nothing.
int gdp_validate(const gdp_problem *p, int i);
// ... and of its initial costs (gdp_problem.f0; GDP_OK when there are none): no NaN / -inf / -0.0, no possible
// overflow.  *f0_live (may be null): they hold something other than zeros.  Allocates nothing.
int gdp_validate_f0(const gdp_problem *p, int i, bool *f0_live);

// Index into GDP_VARIANTS of the register tile ts x r, or -1.
int gdp_find_variant(int ts, int r);
