// serve_rows.hip -- one-workgroup-per-token kernels of the serving engine: embedding, fused residual + layer norm, the
// latent projections' norms + rotary + cache write, the latent query, the output gate.  Statistics and angles are float.
#include "serve_common.h"

static thread_local char g_err[512] = "";
void qsv_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
extern "C" int qsv_version(void) { return 1; }
extern "C" const char* qsv_arch(void) { return "gfx950"; }
extern "C" const char* qsv_last_error(void) { return g_err; }

constexpr int NT = 256;

// ---- embedding ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void embed_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ table,
                                                   const int32_t* __restrict__ tokens, int D) {
    const size_t t = blockIdx.x;
    const T* row = table + (size_t)tokens[t] * D;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float v = ld(row, i);
        x[t * D + i] = v;
        st(h, t * D + i, v);
    }
}
extern "C" int qsv_embed(float* x, void* h, const void* table, const int32_t* tokens, int n, int D, int dtype, void* stream) {
    QSV_REQUIRE(x && h && table && tokens && n >= 0 && D > 0, "qsv_embed: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_embed",
                 hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)table, tokens, D));
    return qsv_launch_status("qsv_embed");
}

// ---- x += layer_norm(y) * w ; h = x -------------------------------------------------------------------------------------------
// Two reductions (mean, then the mean of squared deviations); the row of y is re-read from cache, not held in registers, so any
// width works.
template <typename T>
__global__ __launch_bounds__(NT) void add_layer_norm_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ y,
                                                            const T* __restrict__ w, float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const T* yr = y + t * D;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) s += ld(yr, i);
    const float mean = block_sum<NT>(s, red) / (float)D;
    float q = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float d = ld(yr, i) - mean;
        q += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum<NT>(q, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) {
        const float v = x[t * D + i] + (ld(yr, i) - mean) * inv * ld(w, i);
        x[t * D + i] = v;
        st(h, t * D + i, v);
    }
}
extern "C" int qsv_add_layer_norm(float* x, void* h, const void* y, const void* w, float eps, int n, int D, int dtype,
                                  void* stream) {
    QSV_REQUIRE(x && h && y && w && n >= 0 && D > 0, "qsv_add_layer_norm: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_add_layer_norm",
                 hipLaunchKernelGGL(add_layer_norm_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, x, (T*)h, (const T*)y,
                                    (const T*)w, eps, D));
    return qsv_launch_status("qsv_add_layer_norm");
}

template <typename T>
__global__ __launch_bounds__(NT) void layer_norm_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                             const int32_t* __restrict__ rows, const T* __restrict__ w,
                                                             float eps, int D) {
    __shared__ float red[NT / 64 + 1];
    const size_t r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : (int32_t)r) * D;
    float s = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) s += xr[i];
    const float mean = block_sum<NT>(s, red) / (float)D;
    float q = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) {
        const float d = xr[i] - mean;
        q += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum<NT>(q, red) / (float)D + eps);
    for (int i = threadIdx.x; i < D; i += NT) st(out, r * D + i, (xr[i] - mean) * inv * ld(w, i));
}
extern "C" int qsv_layer_norm_rows(void* out, const float* x, const int32_t* rows, const void* w, float eps, int n, int D,
                                   int dtype, void* stream) {
    QSV_REQUIRE(out && x && w && n >= 0 && D > 0, "qsv_layer_norm_rows: bad arguments");
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_layer_norm_rows",
                 hipLaunchKernelGGL(layer_norm_rows_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (T*)out, x, rows,
                                    (const T*)w, eps, D));
    return qsv_launch_status("qsv_layer_norm_rows");
}

// ---- latent projections: two RMS norms, the rotary key part, the cache row ---------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void latent_prep_kernel(const T* __restrict__ down, int64_t down_stride, int q_off, int q_rank,
                                                         const T* __restrict__ q_w, T* __restrict__ cq, int kv_off, int kv_rank,
                                                         const T* __restrict__ kv_w, int rot_dim, int rot_n,
                                                         const float* __restrict__ rope, T* __restrict__ pool,
                                                         const int64_t* __restrict__ slot, const int32_t* __restrict__ pos,
                                                         float eps) {
    __shared__ float red[NT / 64 + 1];
    const size_t t = blockIdx.x;
    const T* row = down + t * down_stride;
    float s = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += NT) {
        const float v = ld(row, q_off + i);
        s += v * v;
    }
    const float qinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += NT) st(cq, t * q_rank + i, ld(row, q_off + i) * qinv * ld(q_w, i));
    s = 0.f;
    for (int i = threadIdx.x; i < kv_rank; i += NT) {
        const float v = ld(row, kv_off + i);
        s += v * v;
    }
    const float kinv = 1.0f / sqrtf(block_sum<NT>(s, red) / (float)kv_rank + eps);
    T* dst = pool + (size_t)slot[t] * (size_t)(kv_rank + rot_dim);
    for (int i = threadIdx.x; i < kv_rank; i += NT) st(dst, i, ld(row, kv_off + i) * kinv * ld(kv_w, i));
    const int half = rot_n / 2;
    const float* cs = rope ? rope + (size_t)pos[t] * (size_t)rot_n : nullptr;   // [2, half]: cos then sin
    const T* kr = row + kv_off + kv_rank;
    for (int i = threadIdx.x; i < rot_dim; i += NT) {
        float v = ld(kr, i);
        if (i < rot_n) {
            const int p = i >> 1;
            const float c = cs[p], sn = cs[half + p];
            const float u = ld(kr, 2 * p), w2 = ld(kr, 2 * p + 1);
            v = (i & 1) ? (w2 * c + u * sn) : (u * c - w2 * sn);
        }
        st(dst, kv_rank + i, v);
    }
}
extern "C" int qsv_latent_prep(const void* down, int64_t down_stride, int q_off, int q_rank, const void* q_w, void* cq,
                               int kv_off, int kv_rank, const void* kv_w, int rot_dim, int rot_n, const float* rope,
                               void* pool, const int64_t* slot, const int32_t* pos, float eps, int n, int dtype, void* stream) {
    QSV_REQUIRE(down && q_w && cq && kv_w && pool && slot && pos && n >= 0, "qsv_latent_prep: null argument");
    QSV_REQUIRE(q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_n >= 0 && rot_n <= rot_dim && rot_n % 2 == 0,
                "qsv_latent_prep: bad sizes (q_rank %d, kv_rank %d, rot_dim %d, rotated %d)", q_rank, kv_rank, rot_dim, rot_n);
    QSV_REQUIRE(rot_n == 0 || rope, "qsv_latent_prep: rotary part without a cos / sin table");
    QSV_REQUIRE(q_off >= 0 && kv_off >= 0 && q_off + q_rank <= down_stride && kv_off + kv_rank + rot_dim <= down_stride,
                "qsv_latent_prep: the slices do not fit a row of %lld elements", (long long)down_stride);
    if (n == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_latent_prep",
                 hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, (const T*)down, down_stride,
                                    q_off, q_rank, (const T*)q_w, (T*)cq, kv_off, kv_rank, (const T*)kv_w, rot_dim, rot_n, rope,
                                    (T*)pool, slot, pos, eps));
    return qsv_launch_status("qsv_latent_prep");
}

// ---- the query in the latent space: [absorbed part | rotated part], scaled, float ---------------------------------------------
// One workgroup per token, all heads: the absorbed part is a strided gather ([H, T, rank] -> [T, H, rank + rot]), the rotated
// part a handful of values per head.
template <typename T>
__global__ __launch_bounds__(NT) void latent_query_kernel(float* __restrict__ qf, const T* __restrict__ q,
                                                          const T* __restrict__ q_abs, const float* __restrict__ rope,
                                                          const int32_t* __restrict__ pos, float scale, int n_tokens, int H,
                                                          int dim, int rot_dim, int rot_n, int rank) {
    const size_t t = blockIdx.x;
    const int R = rank + rot_dim;
    float* dst = qf + t * H * (size_t)R;
    for (int i = threadIdx.x; i < H * rank; i += NT) {
        const int h = i / rank, c = i - h * rank;
        dst[(size_t)h * R + c] = ld(q_abs, ((size_t)h * n_tokens + t) * (size_t)rank + c) * scale;
    }
    const int half = rot_n / 2;
    const float* cs = rope ? rope + (size_t)pos[t] * (size_t)rot_n : nullptr;
    for (int i = threadIdx.x; i < H * rot_dim; i += NT) {
        const int h = i / rot_dim, c = i - h * rot_dim;
        const T* qr = q + (t * H + h) * (size_t)(dim + rot_dim) + dim;
        float v = ld(qr, c);
        if (c < rot_n) {
            const int p = c >> 1;
            const float co = cs[p], sn = cs[half + p];
            const float u = ld(qr, 2 * p), w2 = ld(qr, 2 * p + 1);
            v = (c & 1) ? (w2 * co + u * sn) : (u * co - w2 * sn);
        }
        dst[(size_t)h * R + rank + c] = v * scale;
    }
}
extern "C" int qsv_latent_query(float* qf, const void* q, const void* q_abs, const float* rope, const int32_t* pos, float scale,
                                int n, int H, int dim, int rot_dim, int rot_n, int rank, int dtype, void* stream) {
    QSV_REQUIRE(qf && q && q_abs && pos && n >= 0 && H > 0 && dim > 0 && rank > 0, "qsv_latent_query: bad arguments");
    QSV_REQUIRE(rot_dim >= 0 && rot_n >= 0 && rot_n <= rot_dim && rot_n % 2 == 0 && (rot_n == 0 || rope),
                "qsv_latent_query: bad rotary sizes (%d of %d)", rot_n, rot_dim);
    if (n == 0) return QSV_OK;
    QSV_REQUIRE((int64_t)n * H < (1ll << 31), "qsv_latent_query: too many (token, head) pairs");
    QSV_DISPATCH(dtype, "qsv_latent_query",
                 hipLaunchKernelGGL(latent_query_kernel<T>, dim3(n), dim3(NT), 0, (hipStream_t)stream, qf, (const T*)q,
                                    (const T*)q_abs, rope, pos, scale, n, H, dim, rot_dim, rot_n, rank));
    return qsv_launch_status("qsv_latent_query");
}

// ---- output gate ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(NT) void sigmoid_gate_kernel(T* __restrict__ o, const T* __restrict__ g, int64_t g_stride, int n) {
    const size_t t = blockIdx.x;
    for (int i = threadIdx.x; i < n; i += NT) {
        const float gate = 1.0f / (1.0f + expf(-ld(g, t * g_stride + i)));
        st(o, t * n + i, ld(o, t * n + i) * gate);
    }
}
extern "C" int qsv_sigmoid_gate(void* o, const void* g, int64_t g_stride, int n_tokens, int n, int dtype, void* stream) {
    QSV_REQUIRE(o && g && n_tokens >= 0 && n > 0 && g_stride >= n, "qsv_sigmoid_gate: bad arguments");
    if (n_tokens == 0) return QSV_OK;
    QSV_DISPATCH(dtype, "qsv_sigmoid_gate",
                 hipLaunchKernelGGL(sigmoid_gate_kernel<T>, dim3(n_tokens), dim3(NT), 0, (hipStream_t)stream, (T*)o, (const T*)g,
                                    g_stride, n));
    return qsv_launch_status("qsv_sigmoid_gate");
}
