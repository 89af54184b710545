// Layer normalisation of the reference's transformer layer for gfx950 (MI355X).
//
// Replaces norm() (inference-engine/src/host/transformer_layer.cpp:50-90) and the residual add that
// follows it in the layer (:476-486 and :601-611).  Numerics follow the reference statement by
// statement: the mean and the variance are accumulated in double and rounded to float, the centred
// value, its square and the three output operations (scale, weight, bias) are separately rounded fp32
// operations (this translation unit is built with -ffp-contract=off), eps = 1e-6.  The only freedom
// taken is the order of the two double-precision sums: a row is summed by 64 lanes and a butterfly
// instead of sequentially, which can move the float mean or variance by one ulp in rare rows.
// The centred value x - mean is computed once and reused (the reference computes the identical
// expression twice).
#include "pimdl_internal.h"

namespace pimdl {

namespace {

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// one wave per row
__global__ __launch_bounds__(256) void layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b,
                                                        const float* __restrict__ residual,
                                                        float* __restrict__ out, uint32_t n, uint32_t d, float eps)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const float* xr = x + (size_t)row * d;
    double s = 0.0;
    for (uint32_t i = lane; i < d; i += 64) s += (double)xr[i];
    const float mean = (float)(wave_sum(s) / (double)d);
    double s2 = 0.0;
    for (uint32_t i = lane; i < d; i += 64) {
        const float v = __fsub_rn(xr[i], mean);
        s2 += (double)__fmul_rn(v, v);
    }
    const float variance = (float)(wave_sum(s2) / (double)d);
    const float scale = 1.0f / sqrtf(__fadd_rn(variance, eps));
    float* o = out + (size_t)row * d;
    const float* r = residual ? residual + (size_t)row * d : nullptr;
    for (uint32_t i = lane; i < d; i += 64) {
        float y = __fsub_rn(xr[i], mean);
        y = __fmul_rn(y, scale);
        y = __fmul_rn(y, w[i]);
        y = __fadd_rn(y, b[i]);
        o[i] = r ? __fadd_rn(r[i], y) : y;
    }
}

// The same for rows of up to 64 * 4 * KV floats with d % 4 == 0 and 16-byte aligned buffers: the row
// is read once with float4 loads and stays in registers for the three passes.  Weight, bias and residual are
// requested together with the row, ahead of the two reductions, so that the wave waits for memory once.
template <int KV>
__global__ __launch_bounds__(256) void layer_norm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ b,
                                                            const float* __restrict__ residual,
                                                            float* __restrict__ out, uint32_t n, uint32_t d, float eps)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const uint32_t d4 = d / 4;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * d);
    float4 xv[KV], wv[KV], bv[KV], rv[KV];
    const float4* r = residual ? reinterpret_cast<const float4*>(residual + (size_t)row * d) : nullptr;
    const float4* w4 = reinterpret_cast<const float4*>(w);
    const float4* b4 = reinterpret_cast<const float4*>(b);
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < d4) {
            xv[k] = xr[i];
            wv[k] = w4[i];
            bv[k] = b4[i];
            if (r) rv[k] = r[i];
        }
    }
    double s = 0.0;
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < d4) {
            s += (double)xv[k].x;
            s += (double)xv[k].y;
            s += (double)xv[k].z;
            s += (double)xv[k].w;
        }
    }
    const float mean = (float)(wave_sum(s) / (double)d);
    double s2 = 0.0;
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        if (lane + 64 * k < d4) {
            xv[k].x = __fsub_rn(xv[k].x, mean);
            xv[k].y = __fsub_rn(xv[k].y, mean);
            xv[k].z = __fsub_rn(xv[k].z, mean);
            xv[k].w = __fsub_rn(xv[k].w, mean);
            s2 += (double)__fmul_rn(xv[k].x, xv[k].x);
            s2 += (double)__fmul_rn(xv[k].y, xv[k].y);
            s2 += (double)__fmul_rn(xv[k].z, xv[k].z);
            s2 += (double)__fmul_rn(xv[k].w, xv[k].w);
        }
    }
    const float variance = (float)(wave_sum(s2) / (double)d);
    const float scale = 1.0f / sqrtf(__fadd_rn(variance, eps));
    float4* o = reinterpret_cast<float4*>(out + (size_t)row * d);
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < d4) {
            float4 y;
            y.x = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].x, scale), wv[k].x), bv[k].x);
            y.y = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].y, scale), wv[k].y), bv[k].y);
            y.z = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].z, scale), wv[k].z), bv[k].z);
            y.w = __fadd_rn(__fmul_rn(__fmul_rn(xv[k].w, scale), wv[k].w), bv[k].w);
            if (r) {
                y.x = __fadd_rn(rv[k].x, y.x);
                y.y = __fadd_rn(rv[k].y, y.y);
                y.z = __fadd_rn(rv[k].z, y.z);
                y.w = __fadd_rn(rv[k].w, y.w);
            }
            o[i] = y;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Unmasked multi-head attention, softmax(q k^T * scale) v per (batch, head), fp32, head_dim 64.
// Replaces the attention step of the reference's layer (src/host/transformer_layer.cpp:211-230:
// KQ = K Q, scale by 1/sqrt(head_dim), soft_max, V KQ, permute back to [n][token_dim]); inputs and
// output stay in the layer's [token][head * 64 + d] order, so no head transposes are needed.
//
// A workgroup = 64 queries of one (batch, head), a wave = 16 of them.  Keys come in chunks of 128
// through LDS (K, then V in the same buffer; V is fetched into registers while the scores are computed from
// K), with the running maximum / sum of a streaming softmax between chunks; 16-key tiles past the end of
// the sequence are skipped.  Both products run on v_mfma_f32_16x16x4_f32, transposed so that nothing has to
// change lanes in between:
//   S^T[key][query]  = K Q^T:  A = K rows (keys), B = this lane's query, 16 steps of 4 dims.  The K
//                      index of lane group g in step s is dim 16 g + s (a sum does not care in which
//                      order its terms are paired), so a lane's operands are 16 consecutive floats.
//                      Result: lane (query j, group g) holds keys 16 kt + 4 g + i of key tile kt.
//   out^T[d][query] += V^T P^T: the B operand of step (kt, i) is that very register (key 16 kt + 4 g + i
//                      from group g), A = V[that key][16 dt + j].  Result: lane (j, g) holds dims
//                      16 dt + 4 g + i of its query: one float4 store per 16-dim tile.
// LDS rows are 68 floats apart: 16 keys x 4 groups (first product) and 16 dims x 4 keys (second) then
// fall into 64 different banks.
// ---------------------------------------------------------------------------------------------
constexpr int AT_KC = 128, AT_PITCH = 68, AT_THREADS = 256;
typedef float v4f __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(AT_THREADS, 3) void attention_hd64_kernel(const float* __restrict__ q,
                                                                   const float* __restrict__ k,
                                                                   const float* __restrict__ v,
                                                                   float* __restrict__ out, uint32_t S,
                                                                   uint32_t in_stride, uint32_t out_stride,
                                                                   float scale)
{
    __shared__ __attribute__((aligned(16))) float kv[AT_KC * AT_PITCH];
    const uint32_t h = blockIdx.y, b = blockIdx.z;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = lane & 15, g = lane >> 4;
    const size_t in_base = (size_t)b * S * in_stride + (size_t)h * 64;
    const uint32_t q_tok = blockIdx.x * 64 + wave * 16 + j;
    const uint32_t q_tok_c = q_tok < S ? q_tok : S - 1;  // rows past S repeat the last query; never stored

    float qreg[16];
    {
        const float* qp = q + in_base + (size_t)q_tok_c * in_stride + 16 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 t = *reinterpret_cast<const float4*>(qp + 4 * i);
            qreg[4 * i + 0] = t.x * scale;
            qreg[4 * i + 1] = t.y * scale;
            qreg[4 * i + 2] = t.z * scale;
            qreg[4 * i + 3] = t.w * scale;
        }
    }
    // 128 keys x 64 floats, zero past S: into registers (eight 16-byte pieces per thread), then into LDS.  The two
    // halves are separate so that V is already on its way while the scores are computed from K.
    constexpr int AT_PIECES = AT_KC * 16 / AT_THREADS;
    auto fetch_chunk = [&](float4 (&r)[AT_PIECES], const float* src, uint32_t kc) {
#pragma unroll
        for (int p = 0; p < AT_PIECES; ++p) {
            const uint32_t i = threadIdx.x + p * AT_THREADS, key = i / 16, c4 = i % 16, tok = kc + key;
            r[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (tok < S) r[p] = *reinterpret_cast<const float4*>(src + in_base + (size_t)tok * in_stride + 4 * c4);
        }
    };
    auto store_chunk = [&](const float4 (&r)[AT_PIECES]) {
#pragma unroll
        for (int p = 0; p < AT_PIECES; ++p) {
            const uint32_t i = threadIdx.x + p * AT_THREADS, key = i / 16, c4 = i % 16;
            *reinterpret_cast<float4*>(&kv[key * AT_PITCH + 4 * c4]) = r[p];
        }
    };
    float4 stage[AT_PIECES];

    float m_run = -__builtin_inff(), l_run = 0.0f;
    v4f o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) o[dt] = (v4f){0.f, 0.f, 0.f, 0.f};

    for (uint32_t kc = 0; kc < S; kc += AT_KC) {
        fetch_chunk(stage, k, kc);
        __syncthreads();  // the previous chunk's V has been consumed
        store_chunk(stage);
        __syncthreads();
        fetch_chunk(stage, v, kc);  // lands while the scores are computed
        v4f s[AT_KC / 16];
#pragma unroll
        for (int kt = 0; kt < AT_KC / 16; ++kt) {
            if (kc + 16 * kt >= S) {  // (uniform) a key tile past the sequence: nothing to compute
                s[kt] = (v4f){0.f, 0.f, 0.f, 0.f};
                continue;
            }
            const float* kp = kv + (16 * kt + j) * AT_PITCH + 16 * g;
            float areg[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 t = *reinterpret_cast<const float4*>(kp + 4 * i);
                areg[4 * i + 0] = t.x;
                areg[4 * i + 1] = t.y;
                areg[4 * i + 2] = t.z;
                areg[4 * i + 3] = t.w;
            }
            v4f acc = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < 16; ++st) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[st], qreg[st], acc, 0, 0, 0);
            s[kt] = acc;
        }
        // keys past S do not take part
        float mx = -__builtin_inff();
#pragma unroll
        for (int kt = 0; kt < AT_KC / 16; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (kc + 16 * kt + 4 * g + i >= S) s[kt][i] = -__builtin_inff();
                mx = fmaxf(mx, s[kt][i]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);  // finite: key kc exists
        const float alpha = __expf(m_run - m_new);  // 0 for the first chunk
        float psum = 0.0f;
#pragma unroll
        for (int kt = 0; kt < AT_KC / 16; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = __expf(s[kt][i] - m_new);
                s[kt][i] = p;
                psum += p;
            }
        psum += __shfl_xor(psum, 16);
        psum += __shfl_xor(psum, 32);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) o[dt] *= alpha;

        __syncthreads();  // every wave is done with K
        store_chunk(stage);
        __syncthreads();
#pragma unroll
        for (int kt = 0; kt < AT_KC / 16; ++kt) {
            if (kc + 16 * kt >= S) continue;  // (uniform) its probabilities are all zero
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float* vp = kv + (16 * kt + 4 * g + i) * AT_PITCH + j;
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vp[16 * dt], s[kt][i], o[dt], 0, 0, 0);
            }
        }
    }
    if (q_tok < S) {
        const float inv = 1.0f / l_run;
        float* op = out + ((size_t)b * S + q_tok) * out_stride + (size_t)h * 64 + 4 * g;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
            *reinterpret_cast<float4*>(op + 16 * dt) = make_float4(o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv);
    }
}

}  // namespace

// Shapes are checked by the caller (head_dim 64, strides multiples of 4 floats, 16-byte aligned pointers).
int launch_attention_hd64(Ctx* ctx, const float* d_q, const float* d_k, const float* d_v, float* d_out, uint32_t batch,
                          uint32_t seq, uint32_t heads, uint32_t in_stride, uint32_t out_stride, float scale)
{
    if (batch == 0 || seq == 0 || heads == 0) return PIMDL_OK;
    hipLaunchKernelGGL(attention_hd64_kernel, dim3((seq + 63) / 64, heads, batch), dim3(AT_THREADS), 0, ctx->stream, d_q,
                       d_k, d_v, d_out, seq, in_stride, out_stride, scale);
    return hip_check(ctx, hipGetLastError(), "attention_hd64_kernel launch");
}

int launch_layer_norm(Ctx* ctx, const float* d_x, const float* d_w, const float* d_b, const float* d_residual,
                      float* d_out, uint32_t n, uint32_t d, float eps)
{
    if (n == 0) return PIMDL_OK;
    const uintptr_t all = reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_w) |
                          reinterpret_cast<uintptr_t>(d_b) | reinterpret_cast<uintptr_t>(d_residual) |
                          reinterpret_cast<uintptr_t>(d_out);
    if (d % 4 == 0 && (all & 15) == 0 && d <= 64 * 4 * 8) {
        if (d <= 64 * 4 * 4)
            hipLaunchKernelGGL(layer_norm_vec_kernel<4>, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b,
                               d_residual, d_out, n, d, eps);
        else
            hipLaunchKernelGGL(layer_norm_vec_kernel<8>, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b,
                               d_residual, d_out, n, d, eps);
        return hip_check(ctx, hipGetLastError(), "layer_norm_vec_kernel launch");
    }
    hipLaunchKernelGGL(layer_norm_kernel, dim3((n + 3) / 4), dim3(256), 0, ctx->stream, d_x, d_w, d_b, d_residual,
                       d_out, n, d, eps);
    return hip_check(ctx, hipGetLastError(), "layer_norm_kernel launch");
}

}  // namespace pimdl
