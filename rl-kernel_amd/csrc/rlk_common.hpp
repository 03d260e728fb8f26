// Shared definitions of the librlk_hip C-ABI implementation (error codes, dtype ids).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/rlk_hip.h"

#ifndef RLK_BK
#define RLK_BK 64  // K elements staged through LDS per pipeline step
#endif

#ifndef RLK_DEFAULT_DZ_BUDGET
#define RLK_DEFAULT_DZ_BUDGET (static_cast<size_t>(512) << 20)  // bytes of one dZ block
#endif

// Records `msg` as the calling thread's last error and returns `code` (always negative).
int rlk_fail(int code, const char* msg);
