// The pipelined attention kernel on int8 Q / K with a K scale per key (or per power of two of keys below 64).
#define PIPE_FN launch_pipe_i8_keys
#define PIPE_MODE MODE_I8
#define PIPE_KEYS true
#define PIPE_QF false
#include "pipe_tu.h"
