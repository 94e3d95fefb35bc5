// Launchers of the software-pipelined attention kernel (attn_pipe.h), one translation unit per family of its
// variants so that they compile side by side: every variant is a kernel of several thousand instructions.
// p.total workgroups of nw * 64 threads (nw = 8 or 4); D = 64 or 128; p.out_f32 picks the output type of the
// 8-bit families.
#pragma once

#include <hip/hip_runtime.h>

#include "attn_fwd.h"

namespace arhip {

void launch_pipe_bf16(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);
void launch_pipe_i8(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);       // K scales over whole tiles
void launch_pipe_i8_keys(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);  // K scales per key
void launch_pipe_i8_qf(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);    // bf16 queries, quantised in the prologue
void launch_pipe_i8_keys_qf(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);  // f32 queries, a scale per query and per key
void launch_pipe_fp8(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);
void launch_pipe_fp8_qf(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);   // bf16 queries, quantised in the prologue
void launch_pipe_fp8_keys(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw);

}  // namespace arhip
