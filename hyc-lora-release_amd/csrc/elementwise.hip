// Element-wise backward operators for gfx950: SiLU backward, SiLU*x2 (forward of the gated
// MLP product) and tanh-GELU backward.  Pure streaming kernels: one 128-bit load per
// operand per lane, four independent chunks in flight per lane.  Loads are ordinary loads (the
// operands were usually written by the kernel before: 5 % faster than non-temporal loads); the
// two-operand kernels also write with ordinary stores (another 5-10 % on [4096 x 11008] and
// [8192 x 11008]), the three-operand backward keeps non-temporal stores (faster at 8192 rows).
//
// The SiLU kernels round to bf16 after every arithmetic operation, as the reference's bf16
// Triton expressions do (operators/silu_kernels.py:42-43, :103-104); the sigmoid itself is
// evaluated in fp32 and rounded once.
#include "hyc_common.hpp"

namespace hyc {

constexpr int kEwThreads = 256;
constexpr int kEwUnroll = 4;

struct SiluBwd {   // o = g * (sig * (1 + x * (1 - sig)))
    __device__ __forceinline__ float operator()(float x, float g) const {
        const float sig = rbf(sigmoidf_(x));
        const float t = rbf(1.0f + rbf(x * rbf(1.0f - sig)));
        return g * rbf(sig * t);
    }
};
struct SiluMul {   // o = (sig(x1) * x1) * x2
    __device__ __forceinline__ float operator()(float x1, float x2) const {
        return rbf(rbf(sigmoidf_(x1)) * x1) * x2;
    }
};
struct SiluOnceMul {   // o = bf16(silu(x1)) * x2 with silu evaluated in fp32 and rounded once, as torch's F.silu
    __device__ __forceinline__ float operator()(float x1, float x2) const {
        return rbf(x1 * sigmoidf_(x1)) * x2;
    }
};
struct GeluBwd {   // d/dx of 0.5 x (1 + tanh(gamma (x + kappa x^3))), times g; fp32 throughout
    __device__ __forceinline__ float operator()(float x, float g) const {
        constexpr float gamma = 0.7978845608028654f, kappa = 0.044715f;
        const float x2 = x * x;
        const float y = gamma * (x + kappa * x2 * x);
        const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * y));   // tanh(y)
        return 0.5f * ((1.0f + t) + x * ((1.0f - t * t) * gamma * (1.0f + 3.0f * kappa * x2))) * g;
    }
};

template <class Op>
__global__ __launch_bounds__(kEwThreads) void binary_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                            uint16_t* __restrict__ o, int64_t n) {
    const Op op;
    const int64_t chunks = n / 8;
    const int64_t c0 = (int64_t)blockIdx.x * (kEwThreads * kEwUnroll) + threadIdx.x;
    u32x4 av[kEwUnroll], bv[kEwUnroll];
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
        const int64_t c = c0 + u * kEwThreads;
        if (c < chunks) {
            av[u] = ld16(a + c * 8);
            bv[u] = ld16(b + c * 8);
        }
    }
#pragma unroll
    for (int u = 0; u < kEwUnroll; ++u) {
        const int64_t c = c0 + u * kEwThreads;
        if (c < chunks) {
            float af[8], bf[8], of[8];
            unpack8(av[u], af);
            unpack8(bv[u], bf);
#pragma unroll
            for (int j = 0; j < 8; ++j) of[j] = op(af[j], bf[j]);
            st16(o + c * 8, pack8(of));
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {       // ragged tail
        const int64_t i = chunks * 8 + threadIdx.x;
        o[i] = f_to_bf(op(bf_to_f(a[i]), bf_to_f(b[i])));
    }
}

// Backward of o = silu(x) * u in one pass: grad_x = silu_backward(x, bf16(g * u)) and
// grad_u = g * silu(x), with silu(x) = bf16(x * sig(x)) evaluated in fp32 and rounded once - what
// torch.nn.functional.silu gives.  The layers that do not use the fused LoRA kernels compute exactly
// this with F.silu, two products and silu_backward
// (models/llama/fused_llama_layer_intra_inter.py:362-381, whose comment asks for this kernel).
__global__ __launch_bounds__(kEwThreads) void silu_mul_bwd_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ u,
                                                                  const uint16_t* __restrict__ g, uint16_t* __restrict__ gx,
                                                                  uint16_t* __restrict__ gu, int64_t n) {
    const SiluBwd dsilu;
    auto one = [&](float xf, float uf, float gf, float& ox, float& ou) {
        ox = dsilu(xf, rbf(gf * uf));
        ou = gf * rbf(xf * sigmoidf_(xf));
    };
    const int64_t chunks = n / 8;
    constexpr int kUnroll = 2;
    const int64_t c0 = (int64_t)blockIdx.x * (kEwThreads * kUnroll) + threadIdx.x;
    u32x4 xv[kUnroll], uv[kUnroll], gv[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
        const int64_t c = c0 + k * kEwThreads;
        if (c < chunks) {
            xv[k] = ld16(x + c * 8);
            uv[k] = ld16(u + c * 8);
            gv[k] = ld16(g + c * 8);
        }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
        const int64_t c = c0 + k * kEwThreads;
        if (c < chunks) {
            float xf[8], uf[8], gf[8], ox[8], ou[8];
            unpack8(xv[k], xf);
            unpack8(uv[k], uf);
            unpack8(gv[k], gf);
#pragma unroll
            for (int j = 0; j < 8; ++j) one(xf[j], uf[j], gf[j], ox[j], ou[j]);
            st16_nt(gx + c * 8, pack8(ox));
            st16_nt(gu + c * 8, pack8(ou));
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {       // ragged tail
        const int64_t i = chunks * 8 + threadIdx.x;
        float ox, ou;
        one(bf_to_f(x[i]), bf_to_f(u[i]), bf_to_f(g[i]), ox, ou);
        gx[i] = f_to_bf(ox);
        gu[i] = f_to_bf(ou);
    }
}

template <class Op>
static int launch_binary(const void* a, const void* b, void* o, int64_t n, void* stream) {
    if (n < 0) return HYC_ERR_SHAPE;
    if (n == 0) return HYC_OK;
    if (!a || !b || !o) return HYC_ERR_NULL;
    if (!aligned16(a) || !aligned16(b) || !aligned16(o)) return HYC_ERR_ALIGN;
    const int64_t blocks = cdiv(cdiv(n, 8), kEwThreads * kEwUnroll);
    if (blocks > INT32_MAX) return HYC_ERR_SHAPE;
    hipLaunchKernelGGL(binary_kernel<Op>, dim3((unsigned)(blocks < 1 ? 1 : blocks)), dim3(kEwThreads), 0,
                       (hipStream_t)stream, (const uint16_t*)a, (const uint16_t*)b, (uint16_t*)o, n);
    return check_launch();
}

}  // namespace hyc

using namespace hyc;

extern "C" int hyc_silu_bwd(const void* x, const void* g, void* out, int64_t n, void* stream) {
    return launch_binary<SiluBwd>(x, g, out, n, stream);
}
extern "C" int hyc_silu_mul(const void* x1, const void* x2, void* out, int64_t n, void* stream) {
    return launch_binary<SiluMul>(x1, x2, out, n, stream);
}
extern "C" int hyc_silu_once_mul(const void* x1, const void* x2, void* out, int64_t n, void* stream) {
    return launch_binary<SiluOnceMul>(x1, x2, out, n, stream);
}
extern "C" int hyc_gelu_bwd(const void* x, const void* g, void* out, int64_t n, void* stream) {
    return launch_binary<GeluBwd>(x, g, out, n, stream);
}
extern "C" int hyc_silu_mul_bwd(const void* x, const void* u, const void* g, void* grad_x, void* grad_u, int64_t n,
                                void* stream) {
    if (n < 0) return HYC_ERR_SHAPE;
    if (n == 0) return HYC_OK;
    if (!x || !u || !g || !grad_x || !grad_u) return HYC_ERR_NULL;
    if (!aligned16(x) || !aligned16(u) || !aligned16(g) || !aligned16(grad_x) || !aligned16(grad_u)) return HYC_ERR_ALIGN;
    const int64_t blocks = cdiv(cdiv(n, 8), kEwThreads * 2);
    if (blocks > INT32_MAX) return HYC_ERR_SHAPE;
    hipLaunchKernelGGL(silu_mul_bwd_kernel, dim3((unsigned)(blocks < 1 ? 1 : blocks)), dim3(kEwThreads), 0, (hipStream_t)stream,
                       (const uint16_t*)x, (const uint16_t*)u, (const uint16_t*)g, (uint16_t*)grad_x, (uint16_t*)grad_u, n);
    return check_launch();
}
