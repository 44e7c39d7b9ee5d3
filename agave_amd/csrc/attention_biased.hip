// Softmax attention with a bias on the scores that depends on the distance between query and
// key, over cache pages stored row by row, for gfx950.  What the callers may combine:
//   * keys and values of different sizes, grouped query heads;
//   * a window (a query at position p sees keys p-W+1 .. p) and first positions that stay
//     visible whatever the window (keys j < keep_first), at their true distances;
//   * the bias: none; a slope per head, score -= slope_h * (p - j); or a table per head over
//     distances, score += table[h][min(p - j, len - 1)] (the host folds any bucketing of
//     distances into the table);
//   * a sink per head: exp(sink_h) is added to the softmax's denominator, with no key or value;
//   * a gate on the output rows: out *= sigmoid(gate), element by element.
// Scores, bias, softmax and the sums over values are 32-bit in every element type.
//
// Cache pages: K [page][kv head][64 rows][hd]; V [page][kv head][64 rows][vd].
// Position j of sequence b lies in row j % 64 of the page in column col(j / 64) of table[b]:
//   col(i) = i < head ? i : head + i - base[b]        (base[b] >= head)
// so the first `head` columns are the pages that hold the kept first positions, and the
// columns after them run from the oldest page the window reaches (base[b]) to the newest.
//
// Kernels: rows into the cache; a plain kernel (a workgroup per token and head, any sizes, both
// element types); a matrix-core kernel for many query rows (bfloat16, sizes in steps of 16).
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

__device__ __forceinline__ int page_col(int pi, int pbase, int head) { return pi < head ? pi : head + pi - pbase; }

// ------------------------------------------------------------------ k and v rows into their pages
template <typename T>
__global__ void kv_append_rows_kernel(const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
                                      T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ table,
                                      int width, const int* __restrict__ base, int head, int n_pages,
                                      const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int nkv, int hd,
                                      int vd) {
    const int t = blockIdx.x;
    const int b = tok_seq[t], p = tok_pos[t];
    const int col = page_col(p / AGAVE_PAGE, base[b], head);
    if (col < 0 || col >= width) return;
    const long pg = table[(size_t)b * width + col];
    if (pg < 0 || pg >= n_pages) return;
    const int row = p % AGAVE_PAGE;
    for (int i = threadIdx.x; i < nkv * hd; i += blockDim.x) {
        const int g = i / hd, d = i % hd;
        k_pages[(((size_t)pg * nkv + g) * AGAVE_PAGE + row) * hd + d] = k[(size_t)t * ldk + i];
    }
    for (int i = threadIdx.x; i < nkv * vd; i += blockDim.x) {
        const int g = i / vd, d = i % vd;
        v_pages[(((size_t)pg * nkv + g) * AGAVE_PAGE + row) * vd + d] = v[(size_t)t * ldv + i];
    }
}

extern "C" int agave_kv_append_rows(int dtype, const void* k, long ldk, const void* v, long ldv, void* k_pages,
                                    void* v_pages, const int* table, int width, const int* base, int head, int n_pages,
                                    const int* tok_seq, const int* tok_pos, int N, int nkv, int hd, int vd,
                                    hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nkv > 0 && hd > 0 && vd > 0, "kv_append_rows: bad sizes N=%d nkv=%d hd=%d vd=%d", N, nkv, hd, vd);
    AGAVE_CHECK(k && v && k_pages && v_pages && table && base && tok_seq && tok_pos && width > 0 && n_pages > 0,
                "kv_append_rows: null buffer or empty table");
    AGAVE_CHECK(ldk >= (long)nkv * hd && ldv >= (long)nkv * vd, "kv_append_rows: a row stride is too small");
    AGAVE_CHECK(head >= 0, "kv_append_rows: negative count of kept pages");
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        kv_append_rows_kernel<float><<<N, 128, 0, stream>>>((const float*)k, ldk, (const float*)v, ldv, (float*)k_pages,
                                                            (float*)v_pages, table, width, base, head, n_pages, tok_seq,
                                                            tok_pos, nkv, hd, vd);
    else if (dtype == AGAVE_BF16)
        kv_append_rows_kernel<bf16><<<N, 128, 0, stream>>>((const bf16*)k, ldk, (const bf16*)v, ldv, (bf16*)k_pages,
                                                           (bf16*)v_pages, table, width, base, head, n_pages, tok_seq,
                                                           tok_pos, nkv, hd, vd);
    else
        AGAVE_CHECK(false, "kv_append_rows: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("kv_append_rows");
    return 0;
}

// ------------------------------------------------------------------ what the attention kernels share
struct BiasedArgs {
    const void* q; long ldq;
    void* out; long ldo;
    const void* gate; long ldg;          // null: no gate
    const void* k_pages; const void* v_pages;
    const int* table; int width; const int* base; int head; int n_pages;
    const int* tok_seq; const int* tok_pos;
    int nh, nkv, hd, vd;
    float scale;
    int window;                          // 0: all earlier keys
    int keep_first;                      // keys j < keep_first stay visible
    int bias_mode;                       // 0 none, 1 slopes, 2 table over distances
    const float* bias; int bias_len;     // slopes [nh], or table [nh][bias_len]
    const float* sink;                   // [nh] or null
};

__device__ __forceinline__ float score_bias(const BiasedArgs& A, int h, int dist) {
    if (A.bias_mode == 1) return -A.bias[h] * (float)dist;
    if (A.bias_mode == 2) return A.bias[(size_t)h * A.bias_len + (dist < A.bias_len ? dist : A.bias_len - 1)];
    return 0.f;
}

// ------------------------------------------------------------------ plain kernel
#define BCHUNK 256           // keys per pass = 4 pages
#define BACC 2               // value size <= 512

template <typename T>
__global__ __launch_bounds__(256) void attn_biased_plain_kernel(BiasedArgs A) {
    __shared__ float qs[512];
    __shared__ float sc[BCHUNK];
    __shared__ long page_of[BCHUNK / AGAVE_PAGE];
    __shared__ float red[16];

    const int tid = threadIdx.x;
    const int nh = A.nh, nkv = A.nkv, hd = A.hd, vd = A.vd;
    const int t = blockIdx.x / nh, h = blockIdx.x % nh;
    const int kvh = h / (nh / nkv);
    const int b = A.tok_seq[t];
    const int p = A.tok_pos[t];
    const int lo = A.window > 0 ? (p - A.window + 1 > 0 ? p - A.window + 1 : 0) : 0;
    const int kept_end = A.keep_first < lo ? A.keep_first : lo;     // keys [0, kept_end) lie before the window
    const int pbase = A.base[b];
    const T* q = (const T*)A.q;
    const T* k_pages = (const T*)A.k_pages;
    const T* v_pages = (const T*)A.v_pages;

    for (int d = tid; d < hd; d += blockDim.x) qs[d] = ld(q + (size_t)t * A.ldq + (size_t)h * hd + d);
    __syncthreads();

    // the sink starts the running maximum and sum: it is one more term of the denominator
    float m = -INFINITY, l = 0.f;
    if (A.sink) {
        m = A.sink[h];
        l = 1.f;
    }
    float acc[BACC] = {0.f, 0.f};

    // two stretches of keys: the kept first positions that the window has left behind, then the window
    for (int part = 0; part < 2; ++part) {
        const int j_lo = part == 0 ? 0 : lo;
        const int j_hi = part == 0 ? kept_end - 1 : p;              // inclusive
        if (j_hi < j_lo) continue;
        for (int c0 = (j_lo / AGAVE_PAGE) * AGAVE_PAGE; c0 <= j_hi; c0 += BCHUNK) {
            if (tid < BCHUNK / AGAVE_PAGE) {
                const int first = c0 + tid * AGAVE_PAGE;
                long pg = -1;
                const int col = page_col(first / AGAVE_PAGE, pbase, A.head);
                if (first <= j_hi && col >= 0 && col < A.width) pg = A.table[(size_t)b * A.width + col];
                if (pg >= A.n_pages) pg = -1;
                page_of[tid] = pg;
            }
            __syncthreads();
            const int j = c0 + tid;
            const long pg = page_of[tid / AGAVE_PAGE];
            const bool valid = j >= j_lo && j <= j_hi && pg >= 0;
            float s = -INFINITY;
            if (valid) {
                const T* kr = k_pages + (((size_t)pg * nkv + kvh) * AGAVE_PAGE + (j % AGAVE_PAGE)) * hd;
                float dot = 0.f;
                for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], ld(kr + d), dot);
                s = dot * A.scale + score_bias(A, h, p - j);
            }
            const float cmax = block_max(s, red);
            const float m_new = fmaxf(m, cmax);
            const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
            const float pr = valid ? expf(s - m_new) : 0.f;
            sc[tid] = pr;
            const float csum = block_sum(pr, red);      // has barriers: sc[] is visible afterwards
            l = l * alpha + csum;
            m = m_new;
#pragma unroll
            for (int a = 0; a < BACC; ++a) {
                const int d = tid + a * 256;
                if (d < vd) {
                    float sum = 0.f;
                    for (int pi = 0; pi < BCHUNK / AGAVE_PAGE; ++pi) {
                        const long vp = page_of[pi];
                        if (vp < 0) continue;
                        const T* vr = v_pages + ((size_t)vp * nkv + kvh) * AGAVE_PAGE * vd + d;
                        for (int r = 0; r < AGAVE_PAGE; ++r) {
                            const float w = sc[pi * AGAVE_PAGE + r];
                            if (w != 0.f) sum = fmaf(w, ld(vr + (size_t)r * vd), sum);   // rows out of range hold w == 0
                        }
                    }
                    acc[a] = acc[a] * alpha + sum;
                }
            }
            __syncthreads();     // sc[] and page_of[] are rewritten by the next pass
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* out = (T*)A.out;
    const T* gate = (const T*)A.gate;
#pragma unroll
    for (int a = 0; a < BACC; ++a) {
        const int d = tid + a * 256;
        if (d < vd) {
            float y = acc[a] * inv;
            if (gate) y *= 1.0f / (1.0f + expf(-ld(gate + (size_t)t * A.ldg + (size_t)h * vd + d)));
            st(out + (size_t)t * A.ldo + (size_t)h * vd + d, y);
        }
    }
}

static int check_biased(const BiasedArgs& A, int N) {
    AGAVE_CHECK(N >= 0 && A.nh > 0 && A.nkv > 0 && A.hd > 0 && A.vd > 0, "attn_biased: bad sizes N=%d nh=%d nkv=%d hd=%d vd=%d", N,
                A.nh, A.nkv, A.hd, A.vd);
    AGAVE_CHECK(A.nh % A.nkv == 0, "attn_biased: %d query heads are not a multiple of %d kv heads", A.nh, A.nkv);
    AGAVE_CHECK(A.hd <= 512 && A.vd <= 256 * BACC, "attn_biased: head sizes %d / %d exceed 512", A.hd, A.vd);
    AGAVE_CHECK(A.ldq >= (long)A.nh * A.hd && A.ldo >= (long)A.nh * A.vd && (!A.gate || A.ldg >= (long)A.nh * A.vd),
                "attn_biased: a row stride is too small");
    AGAVE_CHECK(A.window >= 0 && A.keep_first >= 0 && A.head >= 0, "attn_biased: negative window, kept positions or kept pages");
    AGAVE_CHECK(A.keep_first <= A.head * AGAVE_PAGE, "attn_biased: %d kept positions do not fit %d kept pages", A.keep_first, A.head);
    AGAVE_CHECK(A.bias_mode >= 0 && A.bias_mode <= 2 && (A.bias_mode == 0 || A.bias) && (A.bias_mode != 2 || A.bias_len > 0),
                "attn_biased: bias mode %d without its numbers", A.bias_mode);
    AGAVE_CHECK(A.q && A.out && A.k_pages && A.v_pages && A.table && A.base && A.tok_seq && A.tok_pos && A.width > 0 && A.n_pages > 0,
                "attn_biased: null buffer or empty table");
    AGAVE_CHECK((long)N * A.nh < 2147483647L, "attn_biased: too many (token, head) pairs");
    return 0;
}

extern "C" int agave_attn_biased_plain(int dtype, const void* q, long ldq, void* out, long ldo, const void* gate, long ldg,
                                       const void* k_pages, const void* v_pages, const int* table, int width,
                                       const int* base, int head, int n_pages, const int* tok_seq, const int* tok_pos, int N,
                                       int nh, int nkv, int hd, int vd, float scale, int window, int keep_first,
                                       int bias_mode, const float* bias, int bias_len, const float* sink,
                                       hipStream_t stream) {
    BiasedArgs A{q, ldq, out, ldo, gate, ldg, k_pages, v_pages, table, width, base, head, n_pages, tok_seq, tok_pos,
                 nh, nkv, hd, vd, scale, window, keep_first, bias_mode, bias, bias_len, sink};
    if (check_biased(A, N)) return -1;
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        attn_biased_plain_kernel<float><<<N * nh, 256, 0, stream>>>(A);
    else if (dtype == AGAVE_BF16)
        attn_biased_plain_kernel<bf16><<<N * nh, 256, 0, stream>>>(A);
    else
        AGAVE_CHECK(false, "attn_biased: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("attn_biased_plain");
    return 0;
}
