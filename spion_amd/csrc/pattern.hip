// Pattern discovery on the device: diagonal filter + block pooling in one pass over the score map,
// then (one work-group per map) the quantile threshold, the greedy path walks and the binarised mask.
//
// Restates what the reference does on the host CPU with PyTorch ops and a recursive Python function
// (main_conv_ff.py:35-62 and :254-278; top-k variant main_conv.py:236-256; pool-only main_ff.py:253-272).
#include "common.h"
#include "../../include/spion_hip.h"

#include <algorithm>
#include <cmath>
#include <mutex>

namespace spion {

constexpr int POOL_THREADS = 256;
constexpr int WALK_THREADS = 1024;
constexpr int POOLED_LDS = 36864;  // block grids up to 192 x 192 are walked from LDS (144 KB of the CU's 160)

// pooled[I][J] = (1/bs^2) sum_{i in I, j in J} sum_{t=-hk..hk} A[i+t][j+t]  (zero outside the map).
// Regrouped per source element A[p][q]: its weight is the number of shifts t that land in the block.
// fp64 accumulation in a fixed order, one rounding to fp32.
__global__ __launch_bounds__(POOL_THREADS) void conv_pool_kernel(const float* __restrict__ A, float* __restrict__ pooled,
                                                                 int L, int bs, int nb, int hk) {
    __shared__ double red[POOL_THREADS];
    const int I = blockIdx.y, J = blockIdx.x, map = blockIdx.z;
    const float* Am = A + (size_t)map * L * L;
    const int p0 = max(0, I * bs - hk), p1 = min(L, I * bs + bs + hk);
    const int q0 = max(0, J * bs - hk), q1 = min(L, J * bs + bs + hk);
    const int w = q1 - q0, total = (p1 - p0) * w;
    double acc = 0.0;
    for (int e = threadIdx.x; e < total; e += POOL_THREADS) {
        const int p = p0 + e / w, q = q0 + e % w;
        const int dp = p - I * bs, dq = q - J * bs;  // t must satisfy dp-bs+1 <= t <= dp, same for dq
        const int lo = max(-hk, max(dp, dq) - bs + 1);
        const int hi = min(hk, min(dp, dq));
        if (hi >= lo) acc += (double)Am[(size_t)p * L + q] * (double)(hi - lo + 1);
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int s = POOL_THREADS / 2; s > 0; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) pooled[((size_t)map * nb + I) * nb + J] = (float)(red[0] / ((double)bs * (double)bs));
}

// The same sums for block sizes of at least twice the filter's reach (bs >= 2 hk, so a column feeds its own block
// and at most one neighbour): one work-group per (block row, group of adjacent blocks, map); thread (column, row
// group) walks its share of the bs + 2 hk rows of one column -- consecutive threads read consecutive floats -- and
// keeps two fp64 sums, for the column's own block and for the neighbour it reaches into; one wavefront per block
// then adds the block's partial sums in a fixed order.  Every element is read once per block row it touches
// ((bs + 2 hk) / bs times, the repeats from L2) instead of once per block, and in full rows.
constexpr int CP_COLS = 256, CP_RG = 4;
__global__ __launch_bounds__(CP_COLS* CP_RG) void conv_pool_cols_kernel(const float* __restrict__ A,
                                                                         float* __restrict__ pooled, int L, int bs,
                                                                         int nb, int hk, int gb) {
    __shared__ double part[CP_RG][2][CP_COLS];
    const int I = blockIdx.y, map = blockIdx.z;
    const int Jg = blockIdx.x * gb;  // first block of this group
    const float* Am = A + (size_t)map * L * L;
    const int cc = threadIdx.x % CP_COLS, rg = threadIdx.x / CP_COLS;
    const int ncols = gb * bs + 2 * hk;
    const int q = Jg * bs - hk + cc;
    const int p0 = max(0, I * bs - hk), p1 = min(L, I * bs + bs + hk);
    double a0 = 0.0, a1 = 0.0;
    if (cc < ncols && q >= 0 && q < L) {
        const int J0 = q / bs, c = q - J0 * bs;
        int dq1 = 0;
        bool has1 = false;
        if (c < hk) {  // reaches into the block on the left
            dq1 = c + bs;
            has1 = J0 > 0;
        } else if (c >= bs - hk) {  // ... on the right
            dq1 = c - bs;
            has1 = J0 + 1 < nb;
        }
        auto weight = [&](int dp, int dq) {  // shifts t with dp - t and dq - t inside the block
            const int lo = max(-hk, max(dp, dq) - bs + 1), hi = min(hk, min(dp, dq));
            return max(0, hi - lo + 1);
        };
        const float* col = Am + q;
#pragma unroll 8
        for (int p = p0 + rg; p < p1; p += CP_RG) {
            const int dp = p - I * bs;
            const double v = (double)col[(size_t)p * L];
            a0 += v * (double)weight(dp, c);
            if (has1) a1 += v * (double)weight(dp, dq1);
        }
    }
    part[rg][0][cc] = a0;
    part[rg][1][cc] = a1;
    __syncthreads();
    // wavefront b adds up block b: entries e = 0 .. CP_RG (bs + 2 hk) - 1, lane-strided, then a butterfly
    const int b = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (b < gb && Jg + b < nb) {
        const int base = hk + b * bs, span = bs + 2 * hk;
        double s = 0.0;
        for (int e = lane; e < CP_RG * span; e += 64) {
            const int r = e / span, k = e - r * span - hk;  // column base + k, k = -hk .. bs + hk - 1
            s += part[r][(k < 0 || k >= bs) ? 1 : 0][base + k];
        }
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (lane == 0) pooled[((size_t)map * nb + I) * nb + Jg + b] = (float)(s / ((double)bs * (double)bs));
    }
}

__device__ __forceinline__ uint32_t float_key(float f) {  // order-preserving map to unsigned
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// Key of the element of ascending rank `rank` (0-based) among v[0..N): 8-bit radix select by the whole
// work-group.  hist: 256 ints of LDS, sh: 2 ints of LDS.
__device__ uint32_t block_select(const float* __restrict__ v, int N, int rank, int* hist, int* sh) {
    uint32_t prefix = 0, mask = 0;
    int rem = rank;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < N; i += blockDim.x) {
            uint32_t k = float_key(v[i]);
            if ((k & mask) == prefix) atomicAdd(&hist[(k >> shift) & 255u], 1);
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            // first wavefront: lane l owns bins 4l..4l+3; the bin whose cumulative count first exceeds rem
            const int l = threadIdx.x;
            const int h0 = hist[4 * l], h1 = hist[4 * l + 1], h2 = hist[4 * l + 2], h3 = hist[4 * l + 3];
            const int own = h0 + h1 + h2 + h3;
            int incl = own;
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o, 64);
                if (l >= o) incl += up;
            }
            int c = incl - own;
            const bool last = (l == 63);
            if ((c <= rem && rem < incl) || (last && rem >= incl)) {
                int b = 4 * l;
                if (c + h0 <= rem) { c += h0; ++b;
                    if (c + h1 <= rem) { c += h1; ++b;
                        if (c + h2 <= rem) { c += h2; ++b; } } }
                sh[0] = b;
                sh[1] = rem - c;
            }
        }
        __syncthreads();
        prefix |= (uint32_t)sh[0] << shift;
        mask |= 255u << shift;
        rem = sh[1];
        __syncthreads();
    }
    return prefix;
}

// One work-group per map.
__global__ __launch_bounds__(WALK_THREADS) void threshold_walk_kernel(const float* __restrict__ pooled_all,
                                                                      float* __restrict__ mat_all,
                                                                      float* __restrict__ thresh_out, int nb, int mode,
                                                                      float q, int topk) {
    __shared__ int hist[256];
    __shared__ int sh[2];
    __shared__ int s_cnt;
    __shared__ uint32_t s_min;
    extern __shared__ float s_pooled[];  // N floats when N <= POOLED_LDS (sized by the launch)
    const int map = blockIdx.x, N = nb * nb;
    const float* pooled = pooled_all + (size_t)map * N;
    float* mat = mat_all + (size_t)map * N;

    for (int i = threadIdx.x; i < N; i += blockDim.x) mat[i] = 0.f;
    if (N <= POOLED_LDS) {
        // the select passes and the walkers' dependent neighbour reads then stay in LDS
        for (int i = threadIdx.x; i < N; i += blockDim.x) s_pooled[i] = pooled[i];
        __syncthreads();
        pooled = s_pooled;
    }

    if (mode == SPION_PATTERN_FLOOD) {
        // torch.quantile, linear interpolation, every step in fp32 (main_conv_ff.py:268)
        const float r = q * (float)(N - 1);
        const int lo = (int)floorf(r), hi = (int)ceilf(r);
        const float wgt = r - (float)lo;
        const uint32_t klo = block_select(pooled, N, lo, hist, sh);
        if (threadIdx.x == 0) {
            s_cnt = 0;
            s_min = 0xffffffffu;
        }
        __syncthreads();
        int c = 0;
        uint32_t mn = 0xffffffffu;
        for (int i = threadIdx.x; i < N; i += blockDim.x) {
            uint32_t k = float_key(pooled[i]);
            if (k <= klo) ++c;
            else mn = min(mn, k);
        }
        atomicAdd(&s_cnt, c);
        atomicMin(&s_min, mn);
        __syncthreads();
        const float a = key_float(klo);
        const float b = (hi < s_cnt) ? a : key_float(s_min);  // sorted[hi]
        const float diff = b - a;
        float thresh;
        if (wgt < 0.5f) thresh = a + __fmul_rn(wgt, diff);
        else thresh = b - __fmul_rn(diff, 1.0f - wgt);
        if (threadIdx.x == 0 && thresh_out) thresh_out[map] = thresh;
        __syncthreads();  // mat is zeroed for everyone

        // greedy walks: walker k < nb starts at (0, k), walker nb + k at (k, 0)  (main_conv_ff.py:271-274)
        for (int wk = threadIdx.x; wk < 2 * nb; wk += blockDim.x) {
            int x = wk < nb ? 0 : wk - nb, y = wk < nb ? wk : 0;
            auto at = [&](int xx, int yy) -> float { return (xx < nb && yy < nb) ? pooled[xx * nb + yy] : 0.f; };
            while (x < nb && y < nb) {  // x+1 != nb+1 and y+1 != nb+1 on the sentinel-padded map
                const float Dn = at(x + 1, y), Rt = at(x, y + 1), Dg = at(x + 1, y + 1);
                int nx, ny;
                float val;
                if (Dn > Rt) {
                    if (Dn > Dg) { nx = x + 1; ny = y; val = Dn; }
                    else { nx = x + 1; ny = y + 1; val = Dg; }
                } else {
                    if (Rt > Dg) { nx = x; ny = y + 1; val = Rt; }
                    else { nx = x + 1; ny = y + 1; val = Dg; }
                }
                // ff_mat[nx][ny] = val, later binarised with ff_mat > 0
                if (val > thresh && val > 0.f && nx < nb && ny < nb) mat[nx * nb + ny] = 1.f;
                x = nx;
                y = ny;
            }
        }
    } else {
        // the topk largest pooled blocks (main_conv.py:246-249); ties at the boundary: lower index first
        if (threadIdx.x == 0 && thresh_out) thresh_out[map] = 0.f;
        if (topk > 0) {
            const int k = min(topk, N);
            const uint32_t kk = block_select(pooled, N, N - k, hist, sh);  // k-th largest
            if (threadIdx.x == 0) s_cnt = 0;
            __syncthreads();
            if (threadIdx.x == 0) s_min = 0u;  // number of blocks equal to the k-th largest
            __syncthreads();
            int c = 0, ties = 0;
            for (int i = threadIdx.x; i < N; i += blockDim.x) {
                const uint32_t key = float_key(pooled[i]);
                if (key > kk) {
                    mat[i] = 1.f;
                    ++c;
                } else if (key == kk) {
                    ++ties;
                }
            }
            atomicAdd(&s_cnt, c);
            atomicAdd(&s_min, (uint32_t)ties);
            __syncthreads();
            const int need = k - s_cnt;
            if (need >= (int)s_min) {  // the usual case (one such block): every tie is selected
                for (int i = threadIdx.x; i < N; i += blockDim.x)
                    if (float_key(pooled[i]) == kk) mat[i] = 1.f;
            } else if (threadIdx.x == 0) {
                int left = need;
                for (int i = 0; i < N && left > 0; ++i)
                    if (float_key(pooled[i]) == kk) {
                        mat[i] = 1.f;
                        --left;
                    }
            }
            if (threadIdx.x == 0 && thresh_out) thresh_out[map] = key_float(kk);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nb; i += blockDim.x) mat[i * nb + i] = 1.f;  // main_conv_ff.py:277-278
}

static std::mutex g_ws_mutex;
static float* g_pool_ws = nullptr;
static size_t g_pool_ws_count = 0;

// Mean of the dense phase's probability maps over the batch, then over the heads
// (models/model_transformer.py:136-137: torch.mean(torch.mean(attn, dim=0), dim=0)), read once at HBM rate.
// A is [batch][heads][L][L]; KEY_MAJOR: the maps are stored keys x queries (what the dense kernels write, the
// reference's column-major map) and the mean is written queries x keys, transposed through LDS.
template <bool KEY_MAJOR>
__global__ __launch_bounds__(256) void score_map_mean_kernel(const float* __restrict__ A, int batch, int heads, int L,
                                                             float* __restrict__ Mean, float post) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
    const size_t map = (size_t)L * L;
    const float* a = A + (size_t)(r0 + ty) * L + c0 + tx;
    float hs[4] = {0.f, 0.f, 0.f, 0.f};
    for (int h = 0; h < heads; ++h) {
        float bs[4] = {0.f, 0.f, 0.f, 0.f};
        const float* ah = a + (size_t)h * map;
#pragma unroll 4
        for (int b = 0; b < batch; ++b) {  // 16 loads in flight per thread (measured: 32 are slower)
            const float* ab = ah + (size_t)b * heads * map;
#pragma unroll
            for (int j = 0; j < 4; ++j) bs[j] += __builtin_nontemporal_load(ab + (size_t)8 * j * L);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) hs[j] += bs[j] / (float)batch;
    }
    if (KEY_MAJOR) {
#pragma unroll
        for (int j = 0; j < 4; ++j) tile[ty + 8 * j][tx] = hs[j] / (float)heads * post;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) Mean[(size_t)(c0 + ty + 8 * j) * L + r0 + tx] = tile[tx][ty + 8 * j];
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) Mean[(size_t)(r0 + ty + 8 * j) * L + c0 + tx] = hs[j] / (float)heads * post;
    }
}

// post: factor applied to the result (1 for a plain mean; sums of several maps each are turned into the mean of all
// maps by batch / number of maps summed).
int score_map_mean(const float* Attn, int batch, int heads, int L, int key_major, float* Mean, hipStream_t stream,
                   float post) {
    if (!Attn || !Mean || batch <= 0 || heads <= 0 || L <= 0 || L % 32) {
        set_error("spion_score_map_mean: need Attn, Mean, batch > 0, heads > 0 and seq_len a positive multiple of 32 "
                  "(got %d, %d, %d)", batch, heads, L);
        return 1;
    }
    if (L / 32 > 65535) {
        set_error("spion_score_map_mean: seq_len %d too large", L);
        return 1;
    }
    const dim3 grid(L / 32, L / 32), block(256);
    if (key_major)
        hipLaunchKernelGGL(score_map_mean_kernel<true>, grid, block, 0, stream, Attn, batch, heads, L, Mean, post);
    else
        hipLaunchKernelGGL(score_map_mean_kernel<false>, grid, block, 0, stream, Attn, batch, heads, L, Mean, post);
    return SPION_HIP_OK(hipGetLastError()) ? 0 : 1;
}

// -------------------------------------------------------------------------------------------------
// Dense-to-sparse transition test on the device (main_conv_ff.py:211-242).  After every evaluation the averaged
// score map of each layer is compared with the map kept from an earlier evaluation; the Frobenius distance of the
// two is compared with the previous distance, and once it changed by less than `percent` per cent (after
// truncation to an integer) in every layer the pattern counts as settled.  All state lives in device memory:
//   Prev  [layers][n]  the kept maps;
//   State [2*layers+3] floats: before_distance per layer, change in per cent per layer, then stage
//         (0 = no map kept yet, 1 = a map but no distance yet, 2 = map and distance), the transition flag and a
//         scratch word (whether this call replaces the kept maps).
// The host reads State[2*layers+1] once per evaluation; nothing else comes back.
// -------------------------------------------------------------------------------------------------
constexpr int TRANS_BLOCK = 256;
__global__ __launch_bounds__(TRANS_BLOCK) void transition_partial_kernel(const float* __restrict__ Prev,
                                                                         const float* __restrict__ Cur, long long n,
                                                                         double* __restrict__ Partial) {
    __shared__ double red[TRANS_BLOCK];
    const int layer = blockIdx.y, nblk = gridDim.x;
    const float* a = Prev + (size_t)layer * n;
    const float* b = Cur + (size_t)layer * n;
    double s = 0.0;
    for (long long i = (long long)blockIdx.x * TRANS_BLOCK + threadIdx.x; i < n; i += (long long)nblk * TRANS_BLOCK) {
        const float dlt = a[i] - b[i];  // float difference, as torch computes it
        s += (double)dlt * (double)dlt;
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int o = TRANS_BLOCK / 2; o > 0; o >>= 1) {  // fixed order: the result does not depend on timing
        if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) Partial[(size_t)layer * nblk + blockIdx.x] = red[0];
}

__global__ void transition_decide_kernel(const double* __restrict__ Partial, int nblk, int layers, int percent,
                                         float* __restrict__ State) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    float* before = State;
    float* diff = State + layers;
    float& stage = State[2 * layers];
    float& flag = State[2 * layers + 1];
    float& replace = State[2 * layers + 2];
    replace = 0.f;
    if (flag != 0.f) return;
    if (stage == 0.f) {  // first evaluation: keep the maps, nothing to compare with
        stage = 1.f;
        replace = 1.f;
        return;
    }
    int settled = 0;
    for (int l = 0; l < layers; ++l) {
        double s = 0.0;
        for (int k = 0; k < nblk; ++k) s += Partial[(size_t)l * nblk + k];
        const float dist = (float)sqrt(s);
        if (stage == 1.f) {  // second evaluation: the first distance; the kept maps stay
            before[l] = dist;
            diff[l] = 0.f;
        } else {
            // a previous distance of 0 (two identical maps in a row) gives inf or NaN here, where the
            // reference's int(diff) raises (main_conv_ff.py:228-233): such a layer counts as not settled
            const float dl = (fabsf(dist - before[l]) / before[l]) * 100.f;
            diff[l] = dl;
            before[l] = dist;
            if (isfinite(dl) && dl < 2.0e9f && (int)dl < percent) ++settled;
        }
    }
    if (stage == 1.f) {
        stage = 2.f;
        return;
    }
    if (settled == layers) flag = 1.f;
    else replace = 1.f;
}

__global__ __launch_bounds__(256) void transition_replace_kernel(float* __restrict__ Prev, const float* __restrict__ Cur,
                                                                 long long total, const float* __restrict__ State,
                                                                 int layers) {
    if (State[2 * layers + 2] == 0.f) return;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256)
        Prev[i] = Cur[i];
}

int transition_update(const float* Cur, float* Prev, int layers, long long n, float* State, double* Partial,
                      int partial_blocks, int percent, hipStream_t stream) {
    if (!Cur || !Prev || !State || !Partial || layers <= 0 || n <= 0 || partial_blocks <= 0 || layers > 65535) {
        set_error("spion_transition_update: bad arguments");
        return 1;
    }
    hipLaunchKernelGGL(transition_partial_kernel, dim3(partial_blocks, layers), dim3(TRANS_BLOCK), 0, stream, Prev, Cur,
                       n, Partial);
    hipLaunchKernelGGL(transition_decide_kernel, dim3(1), dim3(64), 0, stream, Partial, partial_blocks, layers, percent,
                       State);
    const long long total = n * layers;
    const int blocks = (int)std::min<long long>((total + 255) / 256, 2048);
    hipLaunchKernelGGL(transition_replace_kernel, dim3(blocks), dim3(256), 0, stream, Prev, Cur, total, State, layers);
    return SPION_HIP_OK(hipGetLastError()) ? 0 : 1;
}

int pattern_generate(const float* Score, int n_maps, int L, int bs, int ksize, int mode, double param, float* Mat,
                     float* Pooled, float* Thresh, hipStream_t stream) {
    if (!Score || !Mat) {
        set_error("spion_pattern_generate: null Score or Mat");
        return 1;
    }
    if (n_maps <= 0 || L <= 0 || bs <= 0 || L % bs) {
        set_error("spion_pattern_generate: need n_maps > 0 and seq_len a positive multiple of block_size (got %d, %d, %d)",
                  n_maps, L, bs);
        return 1;
    }
    if (ksize < 0 || (ksize && ksize % 2 == 0)) {
        set_error("spion_pattern_generate: conv_ksize must be 0 or odd (got %d)", ksize);
        return 1;
    }
    if (mode != SPION_PATTERN_FLOOD && mode != SPION_PATTERN_TOPK) {
        set_error("spion_pattern_generate: unknown mode %d", mode);
        return 1;
    }
    const int nb = L / bs;
    if (nb > 16384 || n_maps > 65535 || nb > 65535) {
        set_error("spion_pattern_generate: block grid %d or map count %d too large", nb, n_maps);
        return 1;
    }
    if (mode == SPION_PATTERN_FLOOD && !(param >= 0.0 && param <= 1.0)) {
        set_error("spion_pattern_generate: quantile %g outside [0, 1]", param);
        return 1;
    }
    // Without a caller's Pooled buffer the pooled maps go to one buffer the library owns: such calls are
    // serialised, and the buffer is reused by the next one as soon as this one has been enqueued -- callers that
    // work on several streams at once pass their own Pooled.
    float* pooled = Pooled;
    std::unique_lock<std::mutex> lock(g_ws_mutex, std::defer_lock);
    if (!pooled) {
        lock.lock();
        const size_t need = (size_t)n_maps * nb * nb;
        if (g_pool_ws_count < need) {
            if (g_pool_ws) (void)hipFree(g_pool_ws);
            g_pool_ws = nullptr;
            g_pool_ws_count = 0;
            if (!SPION_HIP_OK(hipMalloc((void**)&g_pool_ws, sizeof(float) * need))) return 1;
            g_pool_ws_count = need;
        }
        pooled = g_pool_ws;
    }
    const int hk = ksize / 2;
    // blocks per work-group of the streaming kernel (0: block size too small for it, or too wide)
    const int gb = bs >= 2 * hk && bs + 2 * hk <= CP_COLS ? std::min((CP_COLS - 2 * hk) / bs, CP_COLS * CP_RG / 64) : 0;
    if (gb > 0)
        hipLaunchKernelGGL(conv_pool_cols_kernel, dim3((nb + gb - 1) / gb, nb, n_maps), dim3(CP_COLS * CP_RG), 0, stream,
                           Score, pooled, L, bs, nb, hk, gb);
    else
        hipLaunchKernelGGL(conv_pool_kernel, dim3(nb, nb, n_maps), dim3(POOL_THREADS), 0, stream, Score, pooled, L, bs,
                           nb, hk);
    if (!check_launch("conv_pool_kernel")) return 1;
    int topk = 0;
    if (mode == SPION_PATTERN_TOPK) topk = (int)((double)(nb * nb) * param - (double)nb);  // main_conv.py:247
    const size_t walk_lds = (size_t)nb * nb <= (size_t)POOLED_LDS ? sizeof(float) * nb * nb : 0;
    if (walk_lds > 32 * 1024) {  // beyond what a launch may ask for without saying so first
        static std::once_flag once;
        static hipError_t attr_err = hipSuccess;
        std::call_once(once, [] {
            attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(threshold_walk_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, sizeof(float) * POOLED_LDS);
        });
        if (!SPION_HIP_OK(attr_err)) return 1;
    }
    hipLaunchKernelGGL(threshold_walk_kernel, dim3(n_maps), dim3(WALK_THREADS), walk_lds, stream, pooled, Mat, Thresh, nb,
                       mode, (float)param, topk);
    if (!check_launch("threshold_walk_kernel")) return 1;
    return 0;
}

}  // namespace spion
