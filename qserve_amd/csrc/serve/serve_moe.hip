// serve_moe.hip -- mixture of experts: grouped top-k router and the per-token expert products (wave-per-output-row form).
//
// Router scores are float from the first product to the chosen weights.  The expert kernels keep one token's input in LDS
// and let every wave walk output rows with its lanes spread along the reduction (coalesced weight rows).
#include "serve_common.h"

namespace {
constexpr int NT = 256;
constexpr int NW = NT / 64;
constexpr int MAX_EXPERTS = 1024;

// One workgroup per token.  z = router . h by the waves, then one thread does the selection (at most a few thousand steps).
// Ties go to the lower index, for groups and for experts.
template <typename T>
__global__ __launch_bounds__(NT) void moe_route_kernel(int32_t* __restrict__ idx, float* __restrict__ weight,
                                                       const T* __restrict__ h, const T* __restrict__ router, int D, int E,
                                                       int top_k, int G, int keep) {
    __shared__ float s[MAX_EXPERTS];
    __shared__ float gs[MAX_EXPERTS];
    __shared__ unsigned char ok[MAX_EXPERTS];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const T* x = h + t * D;
    for (int e = w; e < E; e += NW) {
        const T* r = router + (size_t)e * D;
        float d = 0.f;
        for (int i = lane; i < D; i += 64) d += ld(r, i) * ld(x, i);
        d = wave_sum(d);
        if (lane == 0) s[e] = d;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    float mx = s[0];
    for (int e = 1; e < E; ++e) mx = fmaxf(mx, s[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) {
        s[e] = expf(s[e] - mx);
        sum += s[e];
    }
    const float inv = 1.0f / sum;
    for (int e = 0; e < E; ++e) s[e] *= inv;
    const int per = E / G;
    for (int g = 0; g < G; ++g) {
        float v = s[g * per];
        for (int e = 1; e < per; ++e) v = fmaxf(v, s[g * per + e]);
        gs[g] = v;
    }
    for (int e = 0; e < E; ++e) ok[e] = 0;
    for (int k = 0; k < keep; ++k) {
        int best = -1;
        for (int g = 0; g < G; ++g)
            if (gs[g] >= 0.f && (best < 0 || gs[g] > gs[best])) best = g;
        gs[best] = -1.f;                            // scores are probabilities: -1 marks a taken group
        for (int e = 0; e < per; ++e) ok[best * per + e] = 1;
    }
    for (int k = 0; k < top_k; ++k) {
        int best = -1;
        for (int e = 0; e < E; ++e)
            if (ok[e] && (best < 0 || s[e] > s[best])) best = e;
        ok[best] = 0;
        idx[t * top_k + k] = best;
        weight[t * top_k + k] = s[best];
    }
}

// One workgroup per (token, chosen expert): act = relu(up_e . h)^2.  Dynamic LDS: D floats.
template <typename T>
__global__ __launch_bounds__(NT) void moe_up_kernel(T* __restrict__ act, const T* __restrict__ h, const T* __restrict__ up,
                                                    const int32_t* __restrict__ idx, int top_k, int D, int ff) {
    extern __shared__ float xs[];
    const size_t slot = blockIdx.x;
    const size_t t = slot / top_k;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < D; i += NT) xs[i] = ld(h, t * D + i);
    __syncthreads();
    const T* W = up + (size_t)idx[slot] * ff * D;
    for (int f = w; f < ff; f += NW) {
        const T* r = W + (size_t)f * D;
        float d = 0.f;
        for (int i = lane; i < D; i += 64) d += ld(r, i) * xs[i];
        d = wave_sum(d);
        if (lane == 0) {
            const float a = fmaxf(d, 0.f);
            st(act, slot * ff + f, a * a);
        }
    }
}

// One workgroup per token: y = sum_k weight_k * down_{e_k} . act_k.  Dynamic LDS: top_k * ff floats.
template <typename T>
__global__ __launch_bounds__(NT) void moe_down_kernel(T* __restrict__ y, const T* __restrict__ act, const T* __restrict__ down,
                                                      const int32_t* __restrict__ idx, const float* __restrict__ weight,
                                                      int top_k, int D, int ff) {
    extern __shared__ float as[];
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top_k * ff; i += NT) as[i] = ld(act, t * top_k * ff + i);
    __syncthreads();
    for (int d = w; d < D; d += NW) {
        float total = 0.f;
        for (int k = 0; k < top_k; ++k) {
            const T* r = down + ((size_t)idx[t * top_k + k] * D + d) * ff;
            float v = 0.f;
            for (int i = lane; i < ff; i += 64) v += ld(r, i) * as[k * ff + i];
            total += weight[t * top_k + k] * wave_sum(v);
        }
        if (lane == 0) st(y, t * D + d, total);
    }
}

// ---- expert-sorted form (many tokens): the products are the vendor's, per expert over contiguous runs of sorted slots; these
// kernels do the permutation in, the activation, and the weighted permutation out -----------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ src,
                                                         const int64_t* __restrict__ order, int div, int width) {
    const size_t i = blockIdx.x;
    const T* s = src + (size_t)(order[i] / div) * width;
    for (int c = threadIdx.x; c < width; c += NT) out[i * width + c] = s[c];
}
template <typename T>
__global__ __launch_bounds__(NT) void relu_sq_kernel(T* __restrict__ a, size_t n) {
    const size_t i = (size_t)blockIdx.x * NT + threadIdx.x;
    if (i < n) {
        const float v = fmaxf(ld(a, i), 0.f);
        st(a, i, v * v);
    }
}
// y[t] = sum_k weight[t, k] * ys[inv[t top_k + k]]
template <typename T>
__global__ __launch_bounds__(NT) void moe_combine_kernel(T* __restrict__ y, const T* __restrict__ ys, const int64_t* __restrict__ inv,
                                                         const float* __restrict__ weight, int top_k, int D) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < D; c += NT) {
        float a = 0.f;
        for (int k = 0; k < top_k; ++k) a += weight[t * top_k + k] * ld(ys, (size_t)inv[t * top_k + k] * D + c);
        st(y, t * D + c, a);
    }
}
}  // namespace

extern "C" int qsv_gather_rows(void* out, const void* src, const int64_t* order, int div, int n_rows, int width, int dtype,
                               void* stream) {
    QSV_REQUIRE(out && src && order && div > 0 && n_rows >= 0 && width > 0, "qsv_gather_rows: bad arguments");
    if (n_rows == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_gather_rows",
                 hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(n_rows), dim3(NT), 0, (hipStream_t)stream, (T*)out, (const T*)src,
                                    order, div, width));
    return qsv_launch_status("qsv_gather_rows");
}
extern "C" int qsv_relu_sq(void* a, int64_t n, int dtype, void* stream) {
    QSV_REQUIRE(a && n >= 0 && n < (1ll << 31) * NT, "qsv_relu_sq: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_relu_sq",
                 hipLaunchKernelGGL(relu_sq_kernel<T>, dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, (hipStream_t)stream, (T*)a,
                                    (size_t)n));
    return qsv_launch_status("qsv_relu_sq");
}
extern "C" int qsv_moe_combine(void* y, const void* ys, const int64_t* inv, const float* weight, int n, int top_k, int D,
                               int dtype, void* stream) {
    QSV_REQUIRE(y && ys && inv && weight && n >= 0 && top_k > 0 && D > 0, "qsv_moe_combine: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_combine",
                 hipLaunchKernelGGL(moe_combine_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)y, (const T*)ys, inv,
                                    weight, top_k, D));
    return qsv_launch_status("qsv_moe_combine");
}

extern "C" int qsv_moe_route(int32_t* idx, float* weight, const void* h, const void* router, int n, int D, int E, int top_k,
                             int G, int keep, int dtype, void* stream) {
    QSV_REQUIRE(idx && weight && h && router && n >= 0 && D > 0, "qsv_moe_route: bad arguments");
    QSV_REQUIRE(E > 0 && E <= MAX_EXPERTS && G > 0 && E % G == 0 && keep > 0 && keep <= G && top_k > 0 &&
                    top_k <= keep * (E / G),
                "qsv_moe_route: %d experts in %d groups, %d groups kept, top %d", E, G, keep, top_k);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_route",
                 hipLaunchKernelGGL(moe_route_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, idx, weight, (const T*)h,
                                    (const T*)router, D, E, top_k, G, keep));
    return qsv_launch_status("qsv_moe_route");
}

extern "C" int qsv_moe_up(void* act, const void* h, const void* up, const int32_t* idx, int n, int top_k, int D, int ff,
                          int dtype, void* stream) {
    QSV_REQUIRE(act && h && up && idx && n >= 0 && top_k > 0 && D > 0 && ff > 0, "qsv_moe_up: bad arguments");
    QSV_REQUIRE((size_t)D * 4 <= 64 * 1024, "qsv_moe_up: width %d does not fit the workgroup's LDS", D);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_up",
                 hipLaunchKernelGGL(moe_up_kernel<T>, dim3(n * top_k), dim3(NT), (size_t)D * 4, (hipStream_t)stream, (T*)act,
                                    (const T*)h, (const T*)up, idx, top_k, D, ff));
    return qsv_launch_status("qsv_moe_up");
}

extern "C" int qsv_moe_down(void* y, const void* act, const void* down, const int32_t* idx, const float* weight, int n,
                            int top_k, int D, int ff, int dtype, void* stream) {
    QSV_REQUIRE(y && act && down && idx && weight && n >= 0 && top_k > 0 && D > 0 && ff > 0, "qsv_moe_down: bad arguments");
    QSV_REQUIRE((size_t)top_k * ff * 4 <= 64 * 1024, "qsv_moe_down: %d x %d activations do not fit the workgroup's LDS", top_k, ff);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_moe_down",
                 hipLaunchKernelGGL(moe_down_kernel<T>, dim3(n), dim3(NT), (size_t)top_k * ff * 4, (hipStream_t)stream, (T*)y,
                                    (const T*)act, (const T*)down, idx, weight, top_k, D, ff));
    return qsv_launch_status("qsv_moe_down");
}
