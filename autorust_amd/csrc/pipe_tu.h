// Body of a pipe_*.hip translation unit: defines PIPE_FN over the variants {D = 64, 128} x {causal, not} x {8, 4 waves}
// of attn_pipe_kernel<., ., PIPE_MODE, false, ., PIPE_KEYS, PIPE_QF>.
#include "attn_pipe.h"
#include "pipe_launch.h"

namespace arhip {
namespace {
template <int D, int NW>
void go(hipStream_t stream, const AttnParams &p, bool causal)
{
    const dim3 grid((unsigned)p.total), block(NW * 64);
    if (causal) hipLaunchKernelGGL((attn_pipe_kernel<D, true, PIPE_MODE, false, NW, PIPE_KEYS, PIPE_QF>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((attn_pipe_kernel<D, false, PIPE_MODE, false, NW, PIPE_KEYS, PIPE_QF>), grid, block, 0, stream, p);
}
}  // namespace

void PIPE_FN(hipStream_t stream, const AttnParams &p, int D, bool causal, int nw)
{
    if (D == 64) {
        if (nw == 4) go<64, 4>(stream, p, causal);
        else go<64, 8>(stream, p, causal);
    } else {
        if (nw == 4) go<128, 4>(stream, p, causal);
        else go<128, 8>(stream, p, causal);
    }
}
}  // namespace arhip
