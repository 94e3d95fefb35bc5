// The pipelined attention kernel on bf16 operands.
#define PIPE_FN launch_pipe_bf16
#define PIPE_MODE MODE_BF16
#define PIPE_KEYS false
#define PIPE_QF false
#include "pipe_tu.h"
