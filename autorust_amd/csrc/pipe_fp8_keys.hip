// The pipelined attention kernel on FP8 E4M3 Q / K with a K scale per key.
#define PIPE_FN launch_pipe_fp8_keys
#define PIPE_MODE MODE_FP8
#define PIPE_KEYS true
#define PIPE_QF false
#include "pipe_tu.h"
