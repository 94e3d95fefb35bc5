// The pipelined int8 attention kernel that quantises its f32 queries row by row in its prologue, K scales per key.
#define PIPE_FN launch_pipe_i8_keys_qf
#define PIPE_MODE MODE_I8
#define PIPE_KEYS true
#define PIPE_QF true
#include "pipe_tu.h"
