// A routed feed-forward (mixture of experts) for gfx950: the choice of experts per token and the
// experts' products over the tokens that chose them.
//
//   s = softmax(z) over all R router outputs (32-bit);  choice score c = s + correction;
//   the R outputs form `groups` equal groups of neighbours, a group's score is its largest c, only
//   the outputs of the `keep` best groups can be chosen; the `top` largest c among them are
//   chosen (the lower index wins a tie); the weight of a chosen output is s * scale.
//   Outputs e >= E are identity experts: their result is the feed-forward's input row itself.
//   Expert e < E: W_down[e] (act(W_gate[e] x) * (W_up[e] x)).
//
// A (token, slot) pair p = t * top + slot names one chosen output.  The plain kernels take the pairs
// as they come (a wave per pair and output column).  The matrix-core kernels take them sorted by
// expert, in tiles of 64 pairs that never span two experts (`route_sort` makes the list and the
// tiles' table on the device, so a step's launches never depend on the choice).
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

#define ROUTE_MAX 1024        // router outputs at most

// ------------------------------------------------------------------ the choice
// One thread per token; `s` [N][R] is scratch that receives the softmax.
__global__ void route_topk_kernel(const float* __restrict__ z, long ldz, const float* __restrict__ correction,
                                  float* __restrict__ s, int N, int R, int groups, int keep, int top, float scale,
                                  int* __restrict__ choice, float* __restrict__ weight) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= N) return;
    const float* zr = z + (size_t)t * ldz;
    float* sr = s + (size_t)t * R;
    float mx = -INFINITY;
    for (int e = 0; e < R; ++e) mx = fmaxf(mx, zr[e]);
    float sum = 0.f;
    for (int e = 0; e < R; ++e) {
        const float w = expf(zr[e] - mx);
        sr[e] = w;
        sum += w;
    }
    const float inv = 1.0f / sum;
    for (int e = 0; e < R; ++e) sr[e] *= inv;
    // groups that may be chosen from: a bit per group (at most 64 groups)
    const int gs = R / groups;
    unsigned long long open = ~0ull;
    if (keep < groups) {
        open = 0ull;
        for (int r = 0; r < keep; ++r) {
            int best = -1;
            float best_v = -INFINITY;
            for (int g = 0; g < groups; ++g) {
                if ((open >> g) & 1ull) continue;
                float gv = -INFINITY;
                for (int e = g * gs; e < (g + 1) * gs; ++e) gv = fmaxf(gv, sr[e] + (correction ? correction[e] : 0.f));
                if (best < 0 || gv > best_v) {
                    best = g;
                    best_v = gv;
                }
            }
            open |= 1ull << best;
        }
    }
    // the `top` best of what is open; what was chosen is marked in the scratch row's sign (s >= 0)
    for (int r = 0; r < top; ++r) {
        int best = -1;
        float best_v = -INFINITY;
        for (int e = 0; e < R; ++e) {
            const float se = sr[e];
            if (se < 0.f || !((open >> (e / gs)) & 1ull)) continue;
            const float c = se + (correction ? correction[e] : 0.f);
            if (best < 0 || c > best_v) {
                best = e;
                best_v = c;
            }
        }
        // (top <= open outputs is checked on the host, so best >= 0)
        choice[(size_t)t * top + r] = best;
        weight[(size_t)t * top + r] = sr[best] * scale;
        sr[best] = -1.0f - sr[best];
    }
}

extern "C" int agave_route_topk(const float* z, long ldz, const float* correction, float* scratch, int N, int R, int groups,
                                int keep, int top, float scale, int* choice, float* weight, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && R > 0 && R <= ROUTE_MAX, "route_topk: %d router outputs (1 to %d)", R, ROUTE_MAX);
    AGAVE_CHECK(groups > 0 && groups <= 64 && R % groups == 0, "route_topk: %d outputs in %d groups (equal groups, at most 64)", R, groups);
    AGAVE_CHECK(keep > 0 && keep <= groups, "route_topk: %d of %d groups kept", keep, groups);
    AGAVE_CHECK(top > 0 && top <= keep * (R / groups), "route_topk: %d chosen of %d that are open", top, keep * (R / groups));
    AGAVE_CHECK(z && scratch && choice && weight && ldz >= R, "route_topk: bad buffers");
    if (N == 0) return 0;
    route_topk_kernel<<<(N + 63) / 64, 64, 0, stream>>>(z, ldz, correction, scratch, N, R, groups, keep, top, scale, choice, weight);
    AGAVE_LAUNCH_CHECK("route_topk");
    return 0;
}

// ------------------------------------------------------------------ activations of the experts' gates
__device__ __forceinline__ float expert_act(float x, int act) {
    switch (act) {
        case 0: { const float c = 0.7978845608028654f; return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x))); }
        case 1: return x / (1.0f + expf(-x));
        case 2: return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
        default: return x > 0.f ? x : 0.f;
    }
}

// ------------------------------------------------------------------ plain products, pair by pair
// act[p][f] = act(W_gate[e] x_t . f) * (W_up[e] x_t . f): a wave per (pair, f), lanes along K
template <typename T>
__global__ __launch_bounds__(256) void routed_gate_up_plain_kernel(const T* __restrict__ x, long ldx, const int* __restrict__ choice,
                                                                   const T* __restrict__ wg, const T* __restrict__ wu,
                                                                   T* __restrict__ act_out, int top, int E, int ff, int K, int act) {
    const int p = blockIdx.x;
    const int e = choice[p];
    if (e < 0 || e >= E) return;
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (f >= ff) return;
    const T* xr = x + (size_t)(p / top) * ldx;
    const T* g = wg + ((size_t)e * ff + f) * K;
    const T* u = wu + ((size_t)e * ff + f) * K;
    float ag = 0.f, au = 0.f;
    for (int k = lane; k < K; k += 64) {
        const float xv = ld(xr + k);
        ag = fmaf(xv, ld(g + k), ag);
        au = fmaf(xv, ld(u + k), au);
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    // (the gate's sum is rounded to the rows' element type before the activation, as a product that
    // writes its rows and an activation kernel that reads them would)
    if (lane == 0) {
        T tg, tu;
        st(&tg, ag);
        st(&tu, au);
        st(act_out + (size_t)p * ff + f, expert_act(ld(&tg), act) * ld(&tu));
    }
}

// y[p][c] = W_down[e][c] . act[p]: a wave per (pair, c), lanes along ff; y is 32-bit
template <typename T>
__global__ __launch_bounds__(256) void routed_down_plain_kernel(const T* __restrict__ act_in, const int* __restrict__ choice,
                                                                const T* __restrict__ wd, float* __restrict__ y, int E, int ff,
                                                                int hidden) {
    const int p = blockIdx.x;
    const int e = choice[p];
    if (e < 0 || e >= E) return;
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= hidden) return;
    const T* a = act_in + (size_t)p * ff;
    const T* w = wd + ((size_t)e * hidden + c) * ff;
    float acc = 0.f;
    for (int f = lane; f < ff; f += 64) acc = fmaf(ld(a + f), ld(w + f), acc);
    acc = wave_sum(acc);
    if (lane == 0) y[(size_t)p * hidden + c] = acc;
}

// out[t] = sum over the token's pairs of weight * (expert row, or the input row for an identity expert) + shared[t].
// `place` (may be null): where pair p's row lies in y (a sorted list); null: at p.
template <typename T>
__global__ void routed_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const int* __restrict__ choice,
                                      const float* __restrict__ weight, const T* __restrict__ x, long ldx,
                                      const T* __restrict__ shared, long lds, T* __restrict__ out, long ldo, int N, int top,
                                      int E, int hidden) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)N * hidden) return;
    const int t = (int)(idx / hidden), c = (int)(idx % hidden);
    float acc = 0.f;
    for (int r = 0; r < top; ++r) {
        const int p = t * top + r;
        const int e = choice[p];
        const float w = weight[p];
        if (e >= E) {
            acc = fmaf(w, ld(x + (size_t)t * ldx + c), acc);
        } else if (e >= 0) {
            const int row = place ? place[p] : p;
            acc = fmaf(w, y[(size_t)row * hidden + c], acc);
        }
    }
    if (shared) acc += ld(shared + (size_t)t * lds + c);
    st(out + (size_t)t * ldo + c, acc);
}

extern "C" int agave_routed_experts_plain(int dtype, const void* x, long ldx, const int* choice, const void* wg, const void* wu,
                                          const void* wd, void* act_rows, float* y, int N, int top, int E, int ff, int hidden,
                                          int act, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && top > 0 && E >= 0 && ff > 0 && hidden > 0, "routed_experts: bad sizes");
    AGAVE_CHECK(act >= 0 && act < 4, "routed_experts: unknown activation %d", act);
    AGAVE_CHECK(x && choice && act_rows && y && ldx >= hidden && (E == 0 || (wg && wu && wd)), "routed_experts: bad buffers");
    AGAVE_CHECK((ff + 3) / 4 <= 65535 && (hidden + 3) / 4 <= 65535, "routed_experts: too many columns for the grid");
    if (N == 0 || E == 0) return 0;
    const dim3 g1(N * top, (ff + 3) / 4), g2(N * top, (hidden + 3) / 4);
    if (dtype == AGAVE_F32) {
        routed_gate_up_plain_kernel<float><<<g1, 256, 0, stream>>>((const float*)x, ldx, choice, (const float*)wg, (const float*)wu,
                                                                   (float*)act_rows, top, E, ff, hidden, act);
        routed_down_plain_kernel<float><<<g2, 256, 0, stream>>>((const float*)act_rows, choice, (const float*)wd, y, E, ff, hidden);
    } else if (dtype == AGAVE_BF16) {
        routed_gate_up_plain_kernel<bf16><<<g1, 256, 0, stream>>>((const bf16*)x, ldx, choice, (const bf16*)wg, (const bf16*)wu,
                                                                  (bf16*)act_rows, top, E, ff, hidden, act);
        routed_down_plain_kernel<bf16><<<g2, 256, 0, stream>>>((const bf16*)act_rows, choice, (const bf16*)wd, y, E, ff, hidden);
    } else
        AGAVE_CHECK(false, "routed_experts: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("routed_experts_plain");
    return 0;
}

extern "C" int agave_routed_combine(int dtype, const float* y, const int* place, const int* choice, const float* weight,
                                    const void* x, long ldx, const void* shared, long lds, void* out, long ldo, int N, int top,
                                    int E, int hidden, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && top > 0 && hidden > 0, "routed_combine: bad sizes");
    AGAVE_CHECK(choice && weight && x && out && (E == 0 || y) && ldx >= hidden && ldo >= hidden && (!shared || lds >= hidden),
                "routed_combine: bad buffers");
    if (N == 0) return 0;
    const long total = (long)N * hidden;
    const int blocks = (int)((total + 255) / 256);
    if (dtype == AGAVE_F32)
        routed_combine_kernel<float><<<blocks, 256, 0, stream>>>(y, place, choice, weight, (const float*)x, ldx, (const float*)shared,
                                                                 lds, (float*)out, ldo, N, top, E, hidden);
    else if (dtype == AGAVE_BF16)
        routed_combine_kernel<bf16><<<blocks, 256, 0, stream>>>(y, place, choice, weight, (const bf16*)x, ldx, (const bf16*)shared,
                                                                lds, (bf16*)out, ldo, N, top, E, hidden);
    else
        AGAVE_CHECK(false, "routed_combine: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("routed_combine");
    return 0;
}
