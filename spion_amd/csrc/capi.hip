// extern "C" surface of libspion_hip.so (declared in include/spion_hip.h) and the error slot.
#include "common.h"

#include <cstdlib>
#include "../../include/spion_hip.h"

namespace spion {

static std::mutex g_err_mutex;
static std::string g_err;
static thread_local HandleHeader* t_handle = nullptr;

void note_current_handle(HandleHeader* h) { t_handle = h; }

// The entry points return void like the reference's, and the reference's Python never asks for an error: so a
// failure is also written to stderr (SPION_QUIET=1 silences it) and SPION_ABORT_ON_ERROR=1 turns it into an abort,
// for callers that would otherwise go on with unwritten output buffers.
void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    {
        std::lock_guard<std::mutex> lock(g_err_mutex);
        g_err = buf;
        if (t_handle) {
            strncpy(t_handle->err, buf, sizeof(t_handle->err) - 1);
            t_handle->err[sizeof(t_handle->err) - 1] = 0;
        }
    }
    const char* quiet = getenv("SPION_QUIET");
    if (!quiet || quiet[0] != '1') fprintf(stderr, "spion_hip: error: %s\n", buf);
    const char* fatal = getenv("SPION_ABORT_ON_ERROR");
    if (fatal && fatal[0] == '1') abort();
}
bool error_pending() {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    return !g_err.empty();
}

// implemented in sparse_attn.hip / dense_attn.hip / pattern.hip
void* sparse_init(int, int, int, int, bool);
void sparse_destroy(void*);
void sparse_forward(void*, const float*, const float*, const float*, const float*, float*, float*, const int*,
                    const int*, int, bool, bool);
void sparse_backward(void*, const float*, const float*, const float*, const float*, const float*, float*, float*,
                     float*, float*, float*, const int*, const int*, int, const float*, bool);
struct HeadLayout {  // as in tile_kernels.h
    long long bstride;
    int hstride;
    int ld;
};
void sparse_forward_strided(void*, const float*, const float*, const float*, const float*, float*, float*, const int*,
                            const int*, int, int, const HeadLayout&, const HeadLayout&);
void sparse_backward_strided(void*, const float*, const float*, const float*, const float*, const float*, const float*,
                             float*, float*, float*, const int*, const int*, int, int, const HeadLayout&,
                             const HeadLayout&, const HeadLayout&);
void dense_forward_strided(void*, const float*, const float*, const float*, const float*, float*, float*, int,
                           const HeadLayout&, const HeadLayout&);
void dense_backward_strided(void*, const float*, const float*, const float*, const float*, const float*, const float*,
                            float*, float*, float*, int, const HeadLayout&, const HeadLayout&, const HeadLayout&);
void sparse_invalidate(void*);
int sparse_register_pattern(void*, const int*, const int*, int, const int*, const int*);
void sparse_forget_pattern(void*, const int*, const int*);
void sparse_backward_noalloc(void*, const float*, const float*, const float*, const float*, const float*, const float*,
                             float*, float*, float*, const int*, const int*, int);
size_t sparse_noalloc_max_rows();
int sparse_last_path(void*);
void sparse_force_element(void*, int);
void sparse_set_bwd_passes(void*, int);
int sparse_debug_counter(void*, int);
int sparse_debug_bf16_plan(const int*, int, int, int, int, int*, int, int*, int, int*, int, int*, int, int*);
void sparse_use_ocache(void*, int);
void* sparse_bf16_init(int, int, int, int);
void sparse_bf16_forward(void*, const void*, const void*, const void*, const float*, void*, float*, const int*,
                         const int*, int);
void sparse_bf16_backward(void*, const void*, const void*, const void*, const float*, const void*, const float*,
                          const void*, void*, void*, void*, const int*, const int*, int);
void sparse_bf16_forward_strided(void*, const void*, const void*, const void*, const float*, void*, float*, const int*,
                                 const int*, int, int, const HeadLayout&, const HeadLayout&);
void sparse_bf16_backward_strided(void*, const void*, const void*, const void*, const float*, const void*, const float*,
                                  const void*, void*, void*, void*, const int*, const int*, int, int, const HeadLayout&,
                                  const HeadLayout&, const HeadLayout&);
int transpose_last2(const float*, float*, int, int, int, hipStream_t);
int transition_update(const float*, float*, int, long long, float*, double*, int, int, hipStream_t);
void* dense_init(int, int, int, bool);
void dense_destroy(void*);
void dense_forward(void*, const float*, const float*, const float*, const float*, float*, float*, bool);
void dense_backward(void*, const float*, const float*, const float*, const float*, const float*, float*, float*,
                    float*);
int pattern_generate(const float*, int, int, int, int, int, double, float*, float*, float*, hipStream_t);
int score_map_mean(const float*, int, int, int, int, float*, hipStream_t, float post = 1.0f);
void dense_forward_strided_mean(void*, const float*, const float*, const float*, const float*, float*, float*, float*, int,
                                const HeadLayout&, const HeadLayout&);

}  // namespace spion

using namespace spion;

extern "C" {

// ---- sparse, bf16 tensors (no reference counterpart) ---------------------------------------------
void* spion_block_bf16_init(int emb_dim, int seq_len, int num_batches, int block_size) {
    note_current_handle(nullptr);
    return sparse_bf16_init(emb_dim, seq_len, num_batches, block_size);
}
void spion_block_bf16_attn_forward(void* h, const void* Q, const void* K, const void* V, const float* Mask, void* Out,
                                   float* Lse, const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_bf16_forward(h, Q, K, V, Mask, Out, Lse, Offsets, Columns, nnz);
}
void spion_block_bf16_attn_backward(void* h, const void* Q, const void* K, const void* V, const float* Mask,
                                    const void* Out, const float* Lse, const void* dO, void* dQ, void* dK, void* dV,
                                    const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_bf16_backward(h, Q, K, V, Mask, Out, Lse, dO, dQ, dK, dV, Offsets, Columns, nnz);
}
void spion_block_bf16_destroy(void* h) { sparse_destroy(h); }
static spion::HeadLayout to_layout(const spion_head_layout* y);
void spion_block_bf16_attn_forward_strided(void* h, const void* Q, const void* K, const void* V, const float* Mask,
                                           void* Out, float* Lse, const int* Offsets, const int* Columns,
                                           const int* SumMat, int nnz, int heads, const spion_head_layout* in,
                                           const spion_head_layout* out) {
    (void)SumMat;
    if (!in || !out) {
        set_error("bf16 attn_forward_strided: null layout argument");
        return;
    }
    sparse_bf16_forward_strided(h, Q, K, V, Mask, Out, Lse, Offsets, Columns, nnz, heads, to_layout(in), to_layout(out));
}
void spion_block_bf16_attn_backward_strided(void* h, const void* Q, const void* K, const void* V, const float* Mask,
                                            const void* Out, const float* Lse, const void* dO, void* dQ, void* dK,
                                            void* dV, const int* Offsets, const int* Columns, const int* SumMat,
                                            int nnz, int heads, const spion_head_layout* in,
                                            const spion_head_layout* out, const spion_head_layout* grad) {
    (void)SumMat;
    if (!in || !out || !grad) {
        set_error("bf16 attn_backward_strided: null layout argument");
        return;
    }
    sparse_bf16_backward_strided(h, Q, K, V, Mask, Out, Lse, dO, dQ, dK, dV, Offsets, Columns, nnz, heads,
                                 to_layout(in), to_layout(out), to_layout(grad));
}

// ---- sparse, no key mask -----------------------------------------------------------------------
void* spion_block_init(int emb_dim, int seq_len, int num_batches, int block_size) {
    note_current_handle(nullptr);
    return sparse_init(emb_dim, seq_len, num_batches, block_size, false);
}
void spion_block_attn_forward(void* h, const float* Q, const float* Kt, const float* V, float* Attn, float* Out,
                              const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_forward(h, Q, Kt, V, nullptr, Attn, Out, Offsets, Columns, nnz, false, false);
}
void spion_block_attn_backward(void* h, const float* Q, const float* K, const float* Vt, const float* P,
                               const float* dO, float* dP, float* dS, float* dQ, float* dK, float* dV,
                               const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_backward(h, Q, K, Vt, P, dO, dP, dS, dQ, dK, dV, Offsets, Columns, nnz, nullptr, false);
}
void spion_block_destroy(void* h) { sparse_destroy(h); }

// ---- sparse, key mask --------------------------------------------------------------------------
void* spion_blockmask_init(int emb_dim, int seq_len, int num_batches, int block_size) {
    note_current_handle(nullptr);
    return sparse_init(emb_dim, seq_len, num_batches, block_size, true);
}
void spion_blockmask_attn_forward(void* h, const float* Q, const float* Kt, const float* V, const float* Mask,
                                  float* Attn, float* Out, const int* Offsets, const int* Columns,
                                  const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_forward(h, Q, Kt, V, Mask, Attn, Out, Offsets, Columns, nnz, true, false);
}
void spion_blockmask_attn_backward(void* h, const float* Q, const float* K, const float* Vt, const float* P,
                                   const float* dO, float* dP, float* dS, float* dQ, float* dK, float* dV,
                                   const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_backward(h, Q, K, Vt, P, dO, dP, dS, dQ, dK, dV, Offsets, Columns, nnz, nullptr, false);
}
void spion_blockmask_destroy(void* h) { sparse_destroy(h); }

// ---- dense phase ---------------------------------------------------------------------------------
void* spion_dense_init(int emb_dim, int seq_len, int num_batches) {
    note_current_handle(nullptr);
    return dense_init(emb_dim, seq_len, num_batches, false);
}
void spion_dense_attn_forward(void* h, const float* Qt, const float* K, const float* Vt, float* Attn, float* Out) {
    dense_forward(h, Qt, K, Vt, nullptr, Attn, Out, false);
}
void spion_dense_attn_backward(void* h, const float* Qt, const float* Kt, const float* V, const float* P,
                               const float* dOt, float* dP, float* dScale, float* dS, float* dQ, float* dK,
                               float* dV) {
    (void)dP;
    (void)dScale;
    (void)dS;
    dense_backward(h, Qt, Kt, V, P, dOt, dQ, dK, dV);
}
void spion_dense_destroy(void* h) { dense_destroy(h); }

void* spion_densemask_init(int emb_dim, int seq_len, int num_batches) {
    note_current_handle(nullptr);
    return dense_init(emb_dim, seq_len, num_batches, true);
}
void spion_densemask_attn_forward(void* h, const float* Qt, const float* K, const float* Vt, const float* Mask,
                                  float* Attn, float* Out) {
    dense_forward(h, Qt, K, Vt, Mask, Attn, Out, true);
}
void spion_densemask_attn_backward(void* h, const float* Qt, const float* Kt, const float* V, const float* P,
                                   const float* dOt, float* dP, float* dScale, float* dS, float* dQ, float* dK,
                                   float* dV) {
    (void)dP;
    (void)dScale;
    (void)dS;
    dense_backward(h, Qt, Kt, V, P, dOt, dQ, dK, dV);
}
void spion_densemask_destroy(void* h) { dense_destroy(h); }

// ---- pattern discovery ---------------------------------------------------------------------------
int spion_pattern_generate(const float* Score, int n_maps, int seq_len, int block_size, int conv_ksize, int mode,
                           double param, float* Mat, float* Pooled, float* Thresh, void* stream) {
    note_current_handle(nullptr);
    return pattern_generate(Score, n_maps, seq_len, block_size, conv_ksize, mode, param, Mat, Pooled, Thresh,
                            static_cast<hipStream_t>(stream));
}

int spion_score_map_mean(const float* Attn, int batch, int heads, int seq_len, int key_major, float* Mean,
                         void* stream) {
    note_current_handle(nullptr);
    return score_map_mean(Attn, batch, heads, seq_len, key_major, Mean, static_cast<hipStream_t>(stream));
}

int spion_transition_update(const float* Cur, float* Prev, int layers, long long elems_per_layer, float* State,
                            double* Partial, int partial_blocks, int percent, void* stream) {
    note_current_handle(nullptr);
    return transition_update(Cur, Prev, layers, elems_per_layer, State, Partial, partial_blocks, percent,
                             static_cast<hipStream_t>(stream));
}

// ---- additions -----------------------------------------------------------------------------------
const char* spion_last_error(void) {
    static thread_local std::string copy;
    std::lock_guard<std::mutex> lock(g_err_mutex);
    copy = g_err;
    return copy.c_str();
}
void spion_clear_error(void) {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    g_err.clear();
}
int spion_error_pending(void) {
    std::lock_guard<std::mutex> lock(g_err_mutex);
    return g_err.empty() ? 0 : 1;
}
const char* spion_handle_error(void* h) {
    HandleHeader* hd = static_cast<HandleHeader*>(h);
    if (!hd || (hd->magic != KIND_SPARSE && hd->magic != KIND_DENSE)) return "not a spion handle";
    return hd->err;
}
void spion_clear_handle_error(void* h) {
    HandleHeader* hd = static_cast<HandleHeader*>(h);
    if (hd && (hd->magic == KIND_SPARSE || hd->magic == KIND_DENSE)) hd->err[0] = 0;
}
void spion_set_stream(void* h, void* stream) {
    HandleHeader* hd = static_cast<HandleHeader*>(h);
    if (!hd || (hd->magic != KIND_SPARSE && hd->magic != KIND_DENSE)) {
        set_error("spion_set_stream: not a spion handle");
        return;
    }
    hd->stream = static_cast<hipStream_t>(stream);
}
void spion_invalidate_pattern(void* h) { sparse_invalidate(h); }
int spion_register_pattern(void* h, const int* Offsets, const int* Columns, int nnz, const int* host_Offsets,
                           const int* host_Columns) {
    return sparse_register_pattern(h, Offsets, Columns, nnz, host_Offsets, host_Columns);
}
void spion_forget_pattern(void* h, const int* Offsets, const int* Columns) { sparse_forget_pattern(h, Offsets, Columns); }
int spion_last_path(void* h) { return sparse_last_path(h); }
void spion_force_element_path(void* h, int on) { sparse_force_element(h, on); }
void spion_set_backward_passes(void* h, int mask) { sparse_set_bwd_passes(h, mask); }
int spion_debug_counter(void* h, int which) { return sparse_debug_counter(h, which); }
int spion_debug_bf16_plan(const int* tile_ptr, int nstrips, int pairs, int num_batches, int lanes, int* items,
                          int cap_items, int* lane_ptr, int cap_ptr, int* lane_ent, int cap_ent, int* longs,
                          int cap_longs, int* counts) {
    return sparse_debug_bf16_plan(tile_ptr, nstrips, pairs, num_batches, lanes, items, cap_items, lane_ptr, cap_ptr,
                                  lane_ent, cap_ent, longs, cap_longs, counts);
}
void spion_use_output_cache(void* h, int on) { sparse_use_ocache(h, on); }
void spion_attn_backward_with_out(void* h, const float* Q, const float* K, const float* Vt, const float* P,
                                  const float* Out, const float* dO, float* dP, float* dS, float* dQ, float* dK,
                                  float* dV, const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_backward(h, Q, K, Vt, P, dO, dP, dS, dQ, dK, dV, Offsets, Columns, nnz, Out, false);
}
void spion_attn_forward_rowmajor(void* h, const float* Q, const float* K, const float* V, const float* Mask,
                                 float* Attn, float* Out, const int* Offsets, const int* Columns, const int* SumMat,
                                 int nnz) {
    (void)SumMat;
    sparse_forward(h, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, Mask != nullptr, true);
}
void spion_attn_backward_rowmajor(void* h, const float* Q, const float* K, const float* V, const float* P,
                                  const float* Out, const float* dO, float* dS, float* dQ, float* dK, float* dV,
                                  const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_backward(h, Q, K, V, P, dO, nullptr, dS, dQ, dK, dV, Offsets, Columns, nnz, Out, true);
}
void spion_attn_backward_noalloc(void* h, const float* Q, const float* K, const float* V, const float* P,
                                 const float* Out, const float* dO, float* dQ, float* dK, float* dV,
                                 const int* Offsets, const int* Columns, const int* SumMat, int nnz) {
    (void)SumMat;
    sparse_backward_noalloc(h, Q, K, V, P, Out, dO, dQ, dK, dV, Offsets, Columns, nnz);
}
long long spion_noalloc_max_rows(void) { return (long long)sparse_noalloc_max_rows(); }
static spion::HeadLayout to_layout(const spion_head_layout* y) {
    return spion::HeadLayout{y->batch_stride, y->head_stride, y->row_stride};
}
void spion_attn_forward_strided(void* h, const float* Q, const float* K, const float* V, const float* Mask, float* Attn,
                                float* Out, const int* Offsets, const int* Columns, const int* SumMat, int nnz,
                                int heads, const spion_head_layout* in, const spion_head_layout* out) {
    (void)SumMat;
    if (!in || !out) {
        set_error("attn_forward_strided: null layout argument");
        return;
    }
    sparse_forward_strided(h, Q, K, V, Mask, Attn, Out, Offsets, Columns, nnz, heads, to_layout(in), to_layout(out));
}
void spion_attn_backward_strided(void* h, const float* Q, const float* K, const float* V, const float* P,
                                 const float* Out, const float* dO, float* dQ, float* dK, float* dV,
                                 const int* Offsets, const int* Columns, const int* SumMat, int nnz, int heads,
                                 const spion_head_layout* in, const spion_head_layout* out,
                                 const spion_head_layout* grad) {
    (void)SumMat;
    if (!in || !out || !grad) {
        set_error("attn_backward_strided: null layout argument");
        return;
    }
    sparse_backward_strided(h, Q, K, V, P, Out, dO, dQ, dK, dV, Offsets, Columns, nnz, heads, to_layout(in),
                            to_layout(out), to_layout(grad));
}
void spion_dense_forward_strided(void* h, const float* Q, const float* K, const float* V, const float* Mask, float* Attn,
                                 float* Out, int heads, const spion_head_layout* in, const spion_head_layout* out) {
    if (!in || !out) {
        set_error("dense attn_forward_strided: null layout argument");
        return;
    }
    dense_forward_strided(h, Q, K, V, Mask, Attn, Out, heads, to_layout(in), to_layout(out));
}
void spion_dense_forward_strided_mean(void* h, const float* Q, const float* K, const float* V, const float* Mask,
                                      float* Attn, float* Out, float* Mean, int heads, const spion_head_layout* in,
                                      const spion_head_layout* out) {
    if (!in || !out) {
        set_error("dense attn_forward_strided_mean: null layout argument");
        return;
    }
    dense_forward_strided_mean(h, Q, K, V, Mask, Attn, Out, Mean, heads, to_layout(in), to_layout(out));
}
void spion_dense_backward_strided(void* h, const float* Q, const float* K, const float* V, const float* P,
                                  const float* Out, const float* dO, float* dQ, float* dK, float* dV, int heads,
                                  const spion_head_layout* in, const spion_head_layout* out,
                                  const spion_head_layout* grad) {
    if (!in || !out || !grad) {
        set_error("dense attn_backward_strided: null layout argument");
        return;
    }
    dense_backward_strided(h, Q, K, V, P, Out, dO, dQ, dK, dV, heads, to_layout(in), to_layout(out), to_layout(grad));
}
int spion_transpose_last2(const float* in, float* out, int batch, int rows, int cols, void* stream) {
    note_current_handle(nullptr);
    return transpose_last2(in, out, batch, rows, cols, static_cast<hipStream_t>(stream));
}
const char* spion_version(void) { return "spion_hip 0.1 (gfx950)"; }

}  // extern "C"
