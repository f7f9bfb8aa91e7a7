// Attention of the stack engine over the paged cache: the MFMA tile kernel for bfloat16 (prefill portions and decoded tokens
// alike), and the dispatch between it and the general kernel of stack_ops.hip (any shape, both element types).
//
// attn_tile_kernel: one workgroup per (16 rows of one entry, head); its NW waves split the key blocks (32 keys each) round-robin -
// key-split waves, so a decoded token with a long context still has NW waves in flight - and merge their partial (max, sum, O)
// through LDS.  Everything is computed TRANSPOSED so that no operand ever changes layout between the two products:
//   S^T = K Q^T      A = K rows straight from the page (key-major, 16 bytes of dim per lane), B = Q^T fragments kept in registers;
//                    the result has one query row per lane column, 4 keys per lane and tile;
//   O^T += V^T P^T   B = P^T, which is exactly what the lane already holds (its 8 scores of the block, as bfloat16);
//                    A = V^T rows, which is why the cache stores values channel-major inside a page ([vdim][page]).
// Both maps of a differential head run side by side and share the V^T fragments.  fp32: scores, soft cap, softmax state, O.
#include "dev_utils.h"
#include "launch_util.h"
#include "stack_kernels.h"

namespace tllm
{
namespace kernels
{
int launch_stack_attention_general(const StackAttnParams& p, hipStream_t stream); // stack_ops.hip

using namespace dev;

namespace
{
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(const uint4& u)
{
    bf16x8 r;
    __builtin_memcpy(&r, &u, 16);
    return r;
}

template <int MAPS, int DK, int VT, int NW>
__global__ __launch_bounds__(NW * 64) void attn_tile_kernel(const StackAttnParams p)
{
    constexpr int D = DK * 32, V = VT * 16;
    extern __shared__ float lds[];
    float* o_part = lds;                          // [NW][MAPS][16][V]
    float* ml_part = lds + NW * MAPS * 16 * V;    // [NW][MAPS][16][2]
    const int e = blockIdx.y, h = blockIdx.z, r0 = blockIdx.x * 16;
    const int count = p.ent_count[e];
    if (r0 >= count)
        return;
    const int first = p.ent_first[e], pos0 = p.ent_pos0[e];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = lane & 15, g4 = lane >> 4;
    const int g = h / (p.heads / p.kv_heads);
    const int page = p.page;
    const int32_t* table = p.block_table + (int64_t) e * p.max_blocks;
    const uint16_t* kp = reinterpret_cast<const uint16_t*>(p.k_pool);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(p.v_pool);

    const int qrow = r0 + col < count ? r0 + col : count - 1;
    const int qpos = pos0 + qrow;
    bf16x8 qf[MAPS][DK];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
            qf[m][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
                reinterpret_cast<const uint16_t*>(p.q) + (((int64_t) (first + qrow) * p.heads + h) * MAPS + m) * D + ks * 32 + 8 * g4));
    const int last_row = r0 + 15 < count ? r0 + 15 : count - 1;
    const int nblk = (pos0 + last_row) / 32 + 1;

    float m_run[MAPS], l_run[MAPS];
    f32x4 acc[MAPS][VT];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        m_run[m] = -INFINITY;
        l_run[m] = 0.f;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
            acc[m][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    for (int kb = w; kb < nblk; kb += NW)
    {
        const int key0 = kb * 32;
        const int blk = table[key0 / page], off = key0 % page;
        uint4 pf[MAPS]; // P^T fragment of the block, 8 bfloat16 per map
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
        {
            f32x4 s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
            {
                s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
                const uint16_t* krow = kp + (((int64_t) blk * (p.kv_heads * MAPS) + g * MAPS + m) * page + off + t * 16 + col) * D + 8 * g4;
#pragma unroll
                for (int ks = 0; ks < DK; ++ks)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(*reinterpret_cast<const uint4*>(krow + ks * 32)), qf[m][ks],
                        s[t], 0, 0, 0);
            }
            float bm = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    float v = s[t][i] * p.scale;
                    if (p.softcap > 0.f)
                        v = p.softcap * tanhf(v / p.softcap);
                    if (key0 + t * 16 + 4 * g4 + i > qpos)
                        v = -INFINITY;
                    s[t][i] = v;
                    bm = fmaxf(bm, v);
                }
            bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
            bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
            const float mn = fmaxf(m_run[m], bm);
            const bool none = mn == -INFINITY; // this row sees no key of this block (nor of any before)
            const float corr = none ? 1.f : __expf(m_run[m] - mn);
            float rs = 0.f;
            float pv[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    const float e_ = none ? 0.f : __expf(s[t][i] - mn);
                    pv[t * 4 + i] = e_;
                    rs += e_;
                }
            rs += __shfl_xor(rs, 16, 64);
            rs += __shfl_xor(rs, 32, 64);
            l_run[m] = l_run[m] * corr + rs;
            m_run[m] = mn;
#pragma unroll
            for (int ct = 0; ct < VT; ++ct)
                acc[m][ct] *= corr;
            pf[m] = make_uint4((uint32_t) f2bf(pv[0]) | ((uint32_t) f2bf(pv[1]) << 16), (uint32_t) f2bf(pv[2]) | ((uint32_t) f2bf(pv[3]) << 16),
                (uint32_t) f2bf(pv[4]) | ((uint32_t) f2bf(pv[5]) << 16), (uint32_t) f2bf(pv[6]) | ((uint32_t) f2bf(pv[7]) << 16));
        }
        // O^T += V^T P^T: slot j of the lane's k group is key 4 g4 + j (j < 4) or 16 + 4 g4 + (j - 4) of the block, in both operands
        const uint16_t* vrow = vp + (((int64_t) blk * p.kv_heads + g) * V + col) * page + off + 4 * g4;
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
        {
            const uint2 lo = *reinterpret_cast<const uint2*>(vrow + (int64_t) ct * 16 * page);
            const uint2 hi = *reinterpret_cast<const uint2*>(vrow + (int64_t) ct * 16 * page + 16);
            const bf16x8 vf = as_bf16x8(make_uint4(lo.x, lo.y, hi.x, hi.y));
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                acc[m][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, as_bf16x8(pf[m]), acc[m][ct], 0, 0, 0);
        }
    }

    // ---- merge of the waves' partials
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        if (g4 == 0)
        {
            ml_part[((w * MAPS + m) * 16 + col) * 2] = m_run[m];
            ml_part[((w * MAPS + m) * 16 + col) * 2 + 1] = l_run[m];
        }
#pragma unroll
        for (int ct = 0; ct < VT; ++ct)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o_part[((w * MAPS + m) * 16 + col) * V + ct * 16 + 4 * g4 + i] = acc[m][ct][i];
    }
    __syncthreads();
    // 16 threads per row at NW = 4 (NW * 4 in general), each a strided set of channels
    constexpr int TPR = NW * 4;
    const int row = threadIdx.x / TPR, sub = threadIdx.x % TPR;
    float wgt[MAPS][NW];
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
    {
        float M = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
            M = fmaxf(M, ml_part[((ww * MAPS + m) * 16 + row) * 2]);
        float L = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
        {
            const float mw = ml_part[((ww * MAPS + m) * 16 + row) * 2];
            wgt[m][ww] = mw == -INFINITY ? 0.f : __expf(mw - M);
            L += wgt[m][ww] * ml_part[((ww * MAPS + m) * 16 + row) * 2 + 1];
        }
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
            wgt[m][ww] /= L;
    }
    constexpr int CPT = (V + TPR - 1) / TPR;
    float o[CPT], ss = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; ++c)
    {
        const int ch = sub + c * TPR;
        o[c] = 0.f;
        if (ch < V)
        {
            float a[MAPS];
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
            {
                a[m] = 0.f;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww)
                    a[m] += wgt[m][ww] * o_part[((ww * MAPS + m) * 16 + row) * V + ch];
            }
            o[c] = MAPS == 2 ? a[0] - p.lambda * a[MAPS - 1] : a[0];
            ss += o[c] * o[c];
        }
    }
    float mul = 1.f;
    if (p.head_norm)
    {
#pragma unroll
        for (int d = 1; d < TPR; d <<= 1)
            ss += __shfl_xor(ss, d, 64);
        mul = p.out_scale / sqrtf(ss / (float) V + p.eps);
    }
    if (r0 + row < count)
    {
        uint16_t* out = reinterpret_cast<uint16_t*>(p.out) + ((int64_t) (first + r0 + row) * p.heads + h) * V;
#pragma unroll
        for (int c = 0; c < CPT; ++c)
            if (sub + c * TPR < V)
                out[sub + c * TPR] = f2bf(o[c] * mul);
    }
}

template <int MAPS, int DK, int VT>
int launch_tile(const StackAttnParams& p, hipStream_t stream)
{
    constexpr int NW = 4;
    const size_t lds = sizeof(float) * ((size_t) NW * MAPS * 16 * VT * 16 + (size_t) NW * MAPS * 16 * 2);
    const void* fn = reinterpret_cast<const void*>(&attn_tile_kernel<MAPS, DK, VT, NW>);
    launch_util::ensure_dynamic_lds(fn, lds);
    const dim3 grid((p.max_count + 15) / 16, p.entries, p.heads);
    hipLaunchKernelGGL((attn_tile_kernel<MAPS, DK, VT, NW>), grid, dim3(NW * 64), lds, stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
    {
        set_error("stack_attention (tile kernel) launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 0;
}

template <int MAPS, int DK>
int launch_tile_v(const StackAttnParams& p, hipStream_t stream)
{
    switch (p.vdim)
    {
    case 32: return launch_tile<MAPS, DK, 2>(p, stream);
    case 64: return launch_tile<MAPS, DK, 4>(p, stream);
    case 128: return launch_tile<MAPS, DK, 8>(p, stream);
    default: return 1;
    }
}

template <int MAPS>
int launch_tile_d(const StackAttnParams& p, hipStream_t stream)
{
    switch (p.dim)
    {
    case 32: return launch_tile_v<MAPS, 1>(p, stream);
    case 64: return launch_tile_v<MAPS, 2>(p, stream);
    case 128: return launch_tile_v<MAPS, 4>(p, stream);
    default: return 1;
    }
}

} // namespace

size_t stack_attn_workspace_floats(int32_t tokens, int32_t heads, int32_t maps, int32_t vdim)
{
    return 0; // the key-split waves of a workgroup merge through LDS
}

// the tile kernel's shapes: bfloat16, dim 32 / 64 / 128, vdim 32 / 64 / 128, pages of a multiple of 32 keys
bool stack_attention_tiled(const StackAttnParams& p)
{
    return p.dtype == DT_BF16 && (p.dim == 32 || p.dim == 64 || p.dim == 128) && (p.vdim == 32 || p.vdim == 64 || p.vdim == 128)
        && p.page % 32 == 0 && p.max_count > 0 && p.entries > 0 && !(reinterpret_cast<uintptr_t>(p.q) & 15)
        && !(reinterpret_cast<uintptr_t>(p.k_pool) & 15) && !(reinterpret_cast<uintptr_t>(p.v_pool) & 7);
}

int launch_stack_attention(const StackAttnParams& p, hipStream_t stream)
{
    if (p.tokens <= 0)
        return 0;
    if (p.heads >= 1 && p.kv_heads >= 1 && p.heads % p.kv_heads == 0 && stack_attention_tiled(p))
    {
        const int rc = p.maps == 2 ? launch_tile_d<2>(p, stream) : (p.maps == 1 ? launch_tile_d<1>(p, stream) : 1);
        if (rc <= 0)
            return rc;
    }
    return launch_stack_attention_general(p, stream);
}

} // namespace kernels
} // namespace tllm
