// The pipelined FP8 attention kernel that quantises its bf16 queries in its prologue.
#define PIPE_FN launch_pipe_fp8_qf
#define PIPE_MODE MODE_FP8
#define PIPE_KEYS false
#define PIPE_QF true
#include "pipe_tu.h"
