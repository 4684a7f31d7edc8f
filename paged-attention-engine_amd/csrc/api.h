// C entry points of the gfx950 kernel library.  Every function launches on the
// given stream, allocates nothing, and returns 0 or a negative code with a
// message behind pae_last_error().  dtype codes: 0 float32, 1 bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {
const char* pae_last_error();
int pae_device_arch(char* out, int cap);  // "gfx950" on the card the kernels are built for

int pae_embedding(int dtype, void* out, const void* table, const int* ids, int num_tokens, int hidden,
                  int vocab, float scale, hipStream_t stream);
int pae_embedding_rows(int dtype, void* residual, const void* table, const int* ids, int num_tokens, int hidden,
                       int vocab, float scale, void* next_rows, const void* next_w, int next_w_is_f32,
                       float* next_stats, hipStream_t stream);
int pae_scaled_rows(void* out, const void* rows, const float* row_stats, int row_stat_tiles, float eps, int num_rows,
                    int hidden, hipStream_t stream);
int pae_logits_finish(float* logits, int64_t n, float scale, float cap, hipStream_t stream);
int pae_add_rmsnorm(int dtype, void* residual, const void* delta, int parts, int64_t part_stride,
                    const void* weight, int w_is_f32, float eps, const int* rows, void* out, int num_rows,
                    int hidden, int write_residual, hipStream_t stream);
int pae_residual_add(int dtype, void* residual, const void* delta, int64_t n, hipStream_t stream);
int pae_copy_i32(int* dst, const int* src, int n, hipStream_t stream);  // src: device or pinned host memory
int pae_scatter_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream);
int pae_rope_table(float* cos_sin, const int* positions, const float* inv_freq, int num_tokens, int half,
                   hipStream_t stream);
int pae_rope_kv_write(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nh, int nkv, int hd, int rot,
                      const void* bias, int b_is_f32, const float* cos_sin, const int* positions, const int* tok_seq, const int* block_tables,
                      int max_blocks, int bs, void* k_cache, void* v_cache, int write_kv, hipStream_t stream);
int pae_swiglu(int dtype, void* out, const void* x, int num_tokens, int inter, int block, hipStream_t stream);
int pae_gemm_plain(int in_dtype, int out_dtype, void* C, int64_t ldc, const void* A, int64_t lda, const void* W,
                   const void* bias, int b_is_f32, int M, int N, int K, hipStream_t stream);
int pae_gemm_skinny(int epilogue, void* out, int64_t ldc, const void* A, int64_t lda, const void* W,
                    const void* bias, int b_is_f32, int M, int N, int K, int splits, int64_t part_stride,
                    float* ticket_parts, int* ticket_counters, const float* row_stats, int row_stat_tiles,
                    float row_eps, void* next_rows, int64_t ld_next, const void* next_w, int next_w_is_f32,
                    float* next_stats, hipStream_t stream);
int pae_skinny_ticket_slots(int M, int N);
int64_t pae_skinny_ticket_floats(int M, int N, int splits);
int pae_gemm_skinny_rope(void* q_out, int64_t ldq, const void* A, int64_t lda, const void* W, const void* bias,
                         int b_is_f32, int M, int K, int nh, int nkv, int hd, int rot, const float* cos_sin,
                         const int* positions, const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                         void* k_cache, void* v_cache, int splits, float* ticket_parts, int* ticket_counters,
                         const float* row_stats, int row_stat_tiles, float row_eps, hipStream_t stream);
int pae_paged_attention_generic(int dtype, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                const void* k_cache, const void* v_cache, const int* positions,
                                const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                                int num_tokens, int nh, int nkv, int hd, float scale, int window,
                                hipStream_t stream);
int pae_attn_decode_split();
int pae_attn_decode_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                         const void* v_cache, const int* dec_work, int num_dec, const int* block_tables,
                         int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window, void* part_acc,
                         void* part_ml, hipStream_t stream);
int pae_attn_prefill_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int* tiles, int num_tiles, const int* positions,
                          const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                          int window, hipStream_t stream);
// A decode step's layers as one resident kernel (see decode_program.hip).
// A caller builds a list of phases in host memory with the put functions (each returns the bytes of
// LDS a quad of four wavefronts needs for the phase, or a negative code), copies it to the device and
// runs it.  pae_program_max_groups() must have been called once on the device, outside any capture.
struct SkinnyRope;
int pae_program_phase_bytes();
int pae_program_barrier_bytes();
int pae_program_max_rows();
int pae_program_max_groups();
int pae_program_lds_limit();
int pae_program_activation_bytes(int rows, int K, int splits);
int pae_program_put_product(void* phases, int index, int epilogue, void* out, int64_t ldc, const void* A, int64_t lda,
                            const void* W, const void* bias, int b_is_f32, int M, int N, int K, int splits,
                            float* ticket_parts, int* ticket_counters, const float* row_stats, int row_stat_tiles,
                            float row_eps, void* next_rows, int64_t ld_next, const void* next_w, int next_w_is_f32,
                            float* next_stats, const SkinnyRope* rope);
int pae_program_put_product_rope(void* phases, int index, void* q_out, int64_t ldq, const void* A, int64_t lda,
                                 const void* W, const void* bias, int b_is_f32, int M, int K, int nh, int nkv, int hd,
                                 int rot, const float* cos_sin, const int* positions, const int* tok_seq,
                                 const int* block_tables, int max_blocks, int bs, void* k_cache, void* v_cache,
                                 int splits, float* ticket_parts, int* ticket_counters, const float* row_stats,
                                 int row_stat_tiles, float row_eps);
int pae_program_put_attention(void* phases, int index, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                              const void* k_cache, const void* v_cache, const int* dec_work, int num_dec,
                              const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                              int window, void* part_acc, void* part_ml);  // two phases: index and index + 1
int pae_program_run(const void* phases, int num_phases, void* barrier, int* host_error, int groups, int quad_lds_bytes,
                    int activation_lds_bytes, int spin_limit, long long* trace, hipStream_t stream);

int pae_sample_chunks(int vocab);
int pae_sample(int* tokens, const float* logits, int64_t ld, const float* temperature, const float* uniform,
               int num_rows, int vocab, float* chunk_max, int* chunk_arg, double* chunk_sum, hipStream_t stream);

// pae_sample without a workspace argument, for callers that cannot allocate device memory (code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
// counterpart in the reference.  The chunk results live in a buffer that is part of the library's
// image on every GPU (16 bytes a slot, PAE_SAMPLE_STATIC_SLOTS slots = 512 KiB, held by each GPU
// the library runs on until the process ends); its device address is looked up once per device, for
// the device that `stream` belongs to (the current device for the null stream), at the first call
// there or by pae_sample_static_prepare() with that device current.  That first lookup asks the
// runtime and must not fall inside a stream capture (it is refused there): prepare, or call once,
// before capturing.  num_rows * pae_sample_chunks(vocab) beyond the slots is refused.  The call
// itself calls no hipMalloc, hipFree or other allocating routine.  Every call on a GPU uses that
// GPU's one buffer: calls that overlap on one GPU (several streams or threads) race, so issue them
// one after the other.  Nothing in the buffer needs clearing between calls: a call writes every
// slot before it reads it.  Same results as pae_sample, bit for bit.
#define PAE_SAMPLE_STATIC_SLOTS 32768
int pae_sample_static_slots();
int pae_sample_static_prepare();
int pae_sample_static(int* tokens, const float* logits, int64_t ld, const float* temperature,
                      const float* uniform, int num_rows, int vocab, hipStream_t stream);
}
