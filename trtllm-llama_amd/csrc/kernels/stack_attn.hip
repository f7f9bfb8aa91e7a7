// Attention of the stack engine over the paged cache: dispatch between the general kernel (stack_ops.hip: any shape, both element
// types) and the tiled forms below.
#include "dev_utils.h"
#include "stack_kernels.h"

namespace tllm
{
namespace kernels
{
int launch_stack_attention_general(const StackAttnParams& p, hipStream_t stream); // stack_ops.hip

size_t stack_attn_workspace_floats(int32_t tokens, int32_t heads, int32_t maps, int32_t vdim)
{
    return 0;
}

int launch_stack_attention(const StackAttnParams& p, hipStream_t stream)
{
    return launch_stack_attention_general(p, stream);
}

} // namespace kernels
} // namespace tllm
