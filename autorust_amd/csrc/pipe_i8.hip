// The pipelined attention kernel on int8 Q / K with K scales over whole 64-key tiles.
#define PIPE_FN launch_pipe_i8
#define PIPE_MODE MODE_I8
#define PIPE_KEYS false
#define PIPE_QF false
#include "pipe_tu.h"
