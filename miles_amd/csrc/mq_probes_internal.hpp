// Host-side plumbing of libmq_probes.so (self-tests and streaming probes; not part of the product library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/miles_quant_probes.h"

enum { MQP_OK = 0, MQP_ERR_ARG = -1, MQP_ERR_HIP = -2 };
int mqp_fail(int code, const char* msg);
int mqp_check_launch(const char* what);
