// Device helpers shared by the kernel files: small vector arithmetic, the value a key starts with,
// the optimizer step (store_push_value of pico-ps/operator/SparsePushOperator.h:448) and its
// application to a table row.
#pragma once

#include "table.h"
#include "probe.h"
#include "user_opt.h"

namespace pshbm {

// ---- small vector helpers ------------------------------------------------------------------
__device__ __forceinline__ float vzero(float) { return 0.0f; }
__device__ __forceinline__ float4 vzero(float4) { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float vadd(float a, float b) { return a + b; }
__device__ __forceinline__ float4 vadd(float4 a, float4 b) {
    return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
// n / d for n*d < 2^32 by one multiply: m = ceil(2^32 / d) (d == 1 handled by m = 2^32).
__device__ __forceinline__ u32 div_small(u32 n, u64 m) { return (u32)(((u64)n * m) >> 32); }
// n / d for any 64-bit n by one multiply-high: m = ceil(2^64 / d), d >= 2.
__device__ __forceinline__ u64 div_big(u64 n, u64 m, u32 d) { return d == 1 ? n : __umul64hi(n, m); }

inline u64 magic32(u32 d) { return ((1ull << 32) + d - 1) / d; }
inline u64 magic64(u32 d) { return d <= 1 ? 0 : (~0ull / d) + 1; }

// The row count an inserting operation leaves, told to the host without a round trip: one 64-bit
// word in page-locked memory, {operation number, rows}. The host adds the sizes of the operations
// it has enqueued since to get an upper bound of the row count.
__device__ __forceinline__ void publish_rows(const TableDev& t, u32 rows) {
    if (t.pub)
        __hip_atomic_store(t.pub, ((unsigned long long)t.op_seq << 32) | rows, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
}

// state blocks of each optimizer, for code specialised by KIND
template <int KIND>
__host__ __device__ constexpr int states_of() {
    return KIND <= 1 ? 0 : KIND == 2 ? 1 : KIND == 3 ? 2 : pshbm_user::STATE_BLOCKS;
}
__device__ __forceinline__ pshbm_user::Hyper user_hyper(const OptParams& o) {
    return pshbm_user::Hyper{o.lr, o.init_acc, o.alpha, o.beta, o.l1, o.l2};
}

// float f of the value a key starts with: weights, then optimizer state
__device__ __forceinline__ float init_float(const TableDev& t, u64 key, u32 f) {
    if (f < t.dim) return t.opt.init_range != 0.0f ? init_weight(t.opt.init_range, key, f) : 0.0f;
    if (t.opt.kind == 2 /*ADAGRAD*/) return t.opt.init_acc;
    if (t.opt.kind == 4 /*USER*/) return pshbm_user::init_state(user_hyper(t.opt), (int)(f / t.dim) - 1);
    return 0.0f;
}
// the weights a pull answers for a key that is not stored (init_store_value + fetch_pull_value of
// pico-ps/operator/SparsePullOperator.h:217,226), column unit c of T
__device__ __forceinline__ float init_pulled(const TableDev& t, u64 key, u32 c, float) {
    return init_weight(t.opt.init_range, key, c);
}
__device__ __forceinline__ float4 init_pulled(const TableDev& t, u64 key, u32 c, float4) {
    return make_float4(init_weight(t.opt.init_range, key, c * 4), init_weight(t.opt.init_range, key, c * 4 + 1),
                       init_weight(t.opt.init_range, key, c * 4 + 2), init_weight(t.opt.init_range, key, c * 4 + 3));
}

// ---- optimizer step ------------------------------------------------------------------------
// One fp32 element; each operation rounds on its own (the file is compiled with
// -ffp-contract=off and correctly rounded divide / sqrt).
template <int KIND>
__device__ __forceinline__ void opt_step(const OptParams& o, float g, float& w, float& s1,
                                         float& s2) {
    if constexpr (KIND == 0) {  // SUM
        w = w + g;
    } else if constexpr (KIND == 1) {  // SGD
        float step = o.lr * g;
        w = w - step;
    } else if constexpr (KIND == 2) {  // ADAGRAD: s1 = accumulator
        float gg = g * g;
        float nn = s1 + gg;
        float num = o.lr * g;
        float step = num / sqrtf(nn);
        s1 = nn;
        w = w - step;
    } else if constexpr (KIND == 4) {  // USER: user_opt.h
        pshbm_user::step(user_hyper(o), g, w, s1, s2);
    } else {  // FTRL: s1 = z, s2 = n
        float gg = g * g;
        float n_new = s2 + gg;
        float sq_new = sqrtf(n_new);
        float sigma = (sq_new - sqrtf(s2)) / o.alpha;
        float sw = sigma * w;
        float z = (s1 + g) - sw;
        float w_new;
        if (fabsf(z) <= o.l1) {
            w_new = 0.0f;
        } else {
            float shrunk = z > 0.0f ? z - o.l1 : z + o.l1;
            float denom = (o.beta + sq_new) / o.alpha + o.l2;
            w_new = -shrunk / denom;
        }
        w = w_new;
        s1 = z;
        s2 = n_new;
    }
}

// N consecutive elements; the optimizer is chosen once, outside the element loop.
template <int N>
__device__ __forceinline__ void opt_step_n(const OptParams& o, const float* g, float* w, float* s1,
                                           float* s2) {
    switch (o.kind) {
        case 0:
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<0>(o, g[e], w[e], s1[e], s2[e]);
            break;
        case 1:
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<1>(o, g[e], w[e], s1[e], s2[e]);
            break;
        case 2:
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<2>(o, g[e], w[e], s1[e], s2[e]);
            break;
        case 3:
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<3>(o, g[e], w[e], s1[e], s2[e]);
            break;
        default:
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<4>(o, g[e], w[e], s1[e], s2[e]);
            break;
    }
}

// Applies the aggregated gradient `g` (columns [col, col+1) in units of T) to row `row`.
template <typename T>
__device__ __forceinline__ void finalize(const TableDev& t, u32 row, u32 col, u32 units, T g) {
    constexpr int N = sizeof(T) / 4;
    if (row >= t.max_rows) return;
    T* r = reinterpret_cast<T*>(t.rows + (u64)row * t.stride_f);
    const int states = t.opt.states;
    T wv = r[col];
    T av = vzero(T()), bv = vzero(T());
    if (states >= 1) av = r[units + col];
    if (states >= 2) bv = r[2 * units + col];
    float* gp = reinterpret_cast<float*>(&g);
    float* wp = reinterpret_cast<float*>(&wv);
    float* ap = reinterpret_cast<float*>(&av);
    float* bp = reinterpret_cast<float*>(&bv);
    opt_step_n<N>(t.opt, gp, wp, ap, bp);
    if (t.dirty && col == 0) t.dirty[row] = 1;
    r[col] = wv;
    if (states >= 1) r[units + col] = av;
    if (states >= 2) r[2 * units + col] = bv;
}

}  // namespace pshbm
