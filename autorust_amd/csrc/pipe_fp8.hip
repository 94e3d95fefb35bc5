// The pipelined attention kernel on FP8 E4M3 Q / K with K scales over whole 64-key tiles.
#define PIPE_FN launch_pipe_fp8
#define PIPE_MODE MODE_FP8
#define PIPE_KEYS false
#define PIPE_QF false
#include "pipe_tu.h"
