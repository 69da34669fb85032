// Host-side glue shared by the entry points: error reporting.
#pragma once
#include "../../include/mi355_attn.h"

// Records `msg` as the calling thread's last error and returns `code`.
int set_error(int code, const char* msg);
