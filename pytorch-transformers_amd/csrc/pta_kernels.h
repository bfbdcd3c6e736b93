// C entry points of the gfx950 kernel library (libpta_kernels.so).
//
// Conventions: every pointer is device memory unless it says "host"; `dtype` is
// 0 for 32-bit float and 1 for bfloat16 and names the type of activations,
// matrices and cache; norm weights and biases are always 32-bit; integer
// arrays are int32; `stream` is a hipStream_t.  Activations are row-major
// [tokens, features].  A function returns 0, or non-zero after storing a message
// that pta_last_error() returns; shapes are checked on the host before a launch.
//
// Key pools have the layout [page, kv_head, 64, head_dim]; value pools are transposed within a page,
// [page, kv_head, head_dim, 64].  `block_table` is [sequences in the step, bt_stride] and lists each
// sequence's pages in order.
#pragma once

#include <stdint.h>

#define PTA_ABI_VERSION 9

#ifdef __cplusplus
extern "C" {
#endif

const char* pta_last_error(void);
int pta_abi_version(void);
int pta_page_size(void);

// out[m, :] = table[ids[m], :]
int pta_embed(void* out, const void* table, const int* ids, int M, int H, int dtype, void* stream);

// out1 = LN(x[rows]) * w1 + b1, and out2 with (w2, b2) if out2 is not null; rows may be null (identity)
int pta_layernorm(void* out1, void* out2, const void* x, const int* rows, const float* w1, const float* b1,
                  const float* w2, const float* b2, int M, int H, float eps, int dtype, void* stream);

// bfloat16 rows: x = round(A + B + add1 + add2 + add3) with A, B products left as 32-bit partial sums [P, M_in, H]
// (summed in order, rounded, bias added and rounded) and up to three tensors (a third only after two); out_x = x,
// out1 = LN(x) * w1 + b1, out2 likewise, each if not null; rows (may be null) selects the M source rows out of M_in
int pta_layernorm_sum(void* out_x, void* out1, void* out2, const float* pa, int Pa, const float* bias_a,
                      const float* pb, int Pb, const float* bias_b, const void* add1, const void* add2,
                      const void* add3, const int* rows, const float* w1, const float* b1, const float* w2, const float* b2, int M_in,
                      int M, int H, float eps, void* stream);
int pta_layernorm_sum_ok(int H);
// rows from which tensors alone (no products, no row selection) are summed and normalised by a wave per row
int pta_layernorm_sum_rows_min(void);

// in place: y = act(round(y + bias)) + add1 + add2; bias, add1, add2 may be null
int pta_epilogue(void* y, int ld_y, const float* bias, const void* add1, const void* add2, int M, int N, int act,
                 int dtype, void* stream);

// How queries and keys are rotated by position, as data (here and in the three launches below that rotate).  The
// first rotary_dim elements of a head are rotated, the rest pass; element pairs are (i, i + rotary_dim / 2)
// (PTA_PAIR_HALF) or (2i, 2i + 1) (PTA_PAIR_INTERLEAVED), each by the angle position * inv_freq[i], cosines and
// sines multiplied by cs_scale.  inv_freq_ld: 0 for one table [rotary_dim / 2] for all tokens, else a table per
// sequence of the step, [sequences, inv_freq_ld], found through token_seq.  A null struct or null inv_freq: no rotation.
enum PtaPairing { PTA_PAIR_HALF = 0, PTA_PAIR_INTERLEAVED = 1 };
typedef struct PtaRotation {
    const float* inv_freq;
    int inv_freq_ld;
    float cs_scale;
    int rotary_dim;
    int pairing;
} PtaRotation;

// A bias on attention scores, as data: slopes[head] * x * scale is added to the score of a query and a key, x being
// the key's position (PTA_BIAS_KEY) or the key's position minus the query's (PTA_BIAS_DISTANCE: 0 for a token's own
// key, negative before it); softmax makes the two equal up to rounding.  bf16 = 1 (PTA_BIAS_KEY only): the position
// and the product are rounded to bfloat16 before the scale, as the reference rounds them
// (src/transformers/models/falcon/modeling_falcon.py:196-198).  A null struct or null slopes: no bias.
enum PtaBiasOf { PTA_BIAS_KEY = 0, PTA_BIAS_DISTANCE = 1 };
typedef struct PtaScoreBias {
    const float* slopes;
    int of;
    int bf16;
    float scale;
} PtaScoreBias;

// split fused qkv rows, add bias, rotate q and k, write q and append k, v.
int pta_qkv_rope_cache(void* q_out, const void* fused, int fused_ld, const float* bias, const PtaRotation* rotation,
                       const int* token_pos, const int* token_seq, const int* block_table, int bt_stride,
                       void* k_pool, void* v_pool, int M, int nh, int nkv, int d, int layout, int write_cache,
                       int dtype, void* stream);

// 0 if the attention kernels (and, with ``rotated``, the kernel that rotates queries and keys) take these sizes, else
// nonzero with the reason in pta_last_error; launches nothing
int pta_attention_sizes_ok(int nh, int nkv, int d, int rotated);

// causal attention of M tokens over their sequences' cache, 32-bit arithmetic
// window: 0, or the number of last positions a token sees (itself included)
// score_bias (null: none): see PtaScoreBias above; with bf16 = 1 the slopes given are expected rounded to bfloat16 too
int pta_attn_generic(void* out, const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                     int bt_stride, const int* token_seq, const int* token_pos, const PtaScoreBias* score_bias,
                     int M, int nh,
                     int nkv, int d, float scale, int window, int dtype, void* stream);

// the same attention for bfloat16 on the matrix cores; cu_tokens [n_seqs + 1] and seq_start [n_seqs] say
// which tokens are whose and how long each sequence was before the step; max_new bounds a sequence's new
// tokens.  n_splits > 1 (decode): keys are cut into ranges of split_size, partial results go to
// po [M, nh, n_splits, d], pm and pl [M, nh, n_splits] (32-bit) and are merged in split order.
// decode_tiles (max_new == 1): column tiles that one wave holds, 1..min(tiles of a KV head, what
// pta_attn_decode_max_tiles gives), or 0 for that most.
int pta_attn_mfma_supported(int d);
// Column tiles (sixteen query heads of one KV head) that one wave of a decode launch can hold at this head size.
int pta_attn_decode_max_tiles(int d);
// decode_waves (max_new == 1): waves of a workgroup that take its range of keys block by block in turn and merge
// their results in LDS (1, 4 or 8; pta_attn_decode_waves_ok says whether the combination with decode_tiles is built).
int pta_attn_decode_waves_ok(int d, int tiles, int waves);
// decode_waves 0 (max_new == 1): the heads of a KV head go to the waves of one workgroup, which share its range of
// keys through LDS (decode_tiles does not apply); pta_attn_decode_shared_ok says whether that is built for this head
// size and this many heads on a KV head.
int pta_attn_decode_shared_ok(int d, int heads_per_kv_head);
// prompt_wide (max_new > 1, head sizes up to 64): 1 workgroups of eight waves, 0 of four, -1 eight where the launch
// still has four workgroups and more for every compute unit.
int pta_attn_mfma(void* out, const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                  int bt_stride, const int* cu_tokens, const int* seq_start, const PtaScoreBias* score_bias,
                  int n_seqs, int max_new, int M, int nh, int nkv, int d, float scale, int split_size, int n_splits, float* po,
                  float* pm, float* pl, int window, int decode_tiles, int decode_waves, int prompt_wide, void* stream);

// C = act(A . W^T + bias) + add1 + add2, all 32-bit, fixed summation order
int pta_gemm_f32(float* C, const float* A, const float* W, const float* bias, const float* add1, const float* add2,
                 int M, int N, int K, int act, void* stream);

// y = act(x . W^T + bias) + add1 + add2 for M <= 64 rows of bfloat16; y is bfloat16, or 32-bit if out_f32.
// variant and waves are tuning knobs (0: chosen from N and K): row tiles per wave, waves per workgroup
int pta_gemm_skinny_bf16(void* y, const void* x, const void* W, const float* bias, const void* add1, const void* add2,
                         int M, int N, int K, int act, int out_f32, int variant, int waves, void* stream);

// two such products of one launch, both [M, *] in bfloat16 with one K (a block's two input projections)
int pta_gemm_skinny_pair_bf16(void* y1, const void* x1, const void* W1, const float* bias1, int N1, int act1, void* y2,
                              const void* x2, const void* W2, const float* bias2, int N2, int act2, int M, int K,
                              void* stream);

// the pair launch of a decode step (M <= 16) whose first product is a fused query_key_value projection: its rows
// are split, rotated and written as queries [M, heads, d] and into the cache pages, as pta_qkv_rope_cache leaves
// them; head sizes that are multiples of 32
int pta_gemm_skinny_pair_qkv_bf16(void* q_out, const void* x1, const void* W1, const float* bias1,
                                  const PtaRotation* rotation, const int* token_pos,
                                  const int* token_seq,
                                  const int* block_table, int bt_stride, void* k_pool, void* v_pool, int nh, int nkv,
                                  int d, int layout, int write_cache, void* y2, const void* x2, const void* W2,
                                  const float* bias2, int N2, int act2, int M, int K, void* stream);

// The same product for a batch of up to 128 rows that shares x through LDS and may split K over workgroups:
// `part` is a 32-bit workspace [parts, M, N], needed when parts > 1 or reduce = 0.  rt (row tiles per wave),
// parts, stage_blocks (64-element blocks of K per stage) and depth (stages in flight) are tuning knobs (0:
// chosen from N and K alone); pta_gemm_splitk_parts tells the number of ranges that choice gives.
// With reduce = 0 the product is left as the partial sums (y may be null; bias, act and additions are not
// applied).  Ranges that would be empty are dropped: ceil(nkb / ceil(nkb / parts)) remain, nkb = ceil(K / 64).
int pta_gemm_splitk_bf16(void* y, float* part, const void* x, const void* W, const float* bias, const void* add1,
                         const void* add2, int M, int N, int K, int act, int out_f32, int rt, int parts,
                         int stage_blocks, int depth, int reduce, void* stream);
int pta_gemm_splitk_parts(int N, int K, int parts, int rt);
// two products of one launch, both left as partial sums: part1 [parts1, M, N1], part2 [parts2, M, N2], with the
// ranges pta_gemm_splitk_pair_parts gives
int pta_gemm_splitk_pair_parts(int N1, int K1, int N2, int K2, int M, int* parts1, int* parts2);

// the pair run to the end with the first product a fused query_key_value projection (N1 = (nh + 2 nkv) d rows of
// W1): queries rotated in q_out [M, nh, d], keys and values in the cache pages, as pta_qkv_rope_cache leaves them
int pta_gemm_splitk_pair_reduced_qkv_bf16(void* q_out, float* part1, const void* x1, const void* W1, const float* bias1,
                                          int K1, const PtaRotation* rotation,
                                          const int* token_pos,
                                          const int* token_seq, const int* block_table, int bt_stride, void* k_pool,
                                          void* v_pool, int nh, int nkv, int d, int layout, int write_cache, void* y2,
                                          float* part2, const void* x2, const void* W2, const float* bias2, int N2, int K2,
                                          int act2, int M, void* stream);
// such a projection on its own: part [pta_gemm_splitk_parts(N, K, 0, 0), M, N] is the workspace
int pta_gemm_splitk_reduced_qkv_bf16(void* q_out, float* part, const void* x, const void* W, const float* bias, int K,
                                     const PtaRotation* rotation, const int* token_pos,
                                     const int* token_seq,
                                     const int* block_table, int bt_stride, void* k_pool, void* v_pool, int nh, int nkv,
                                     int d, int layout, int write_cache, int M, void* stream);

// a frequency table per sequence of the step, out [n_seqs, d/2], for frequencies that follow the sequence's length
// after the step (seq_start[s] + its tokens): 1 / base^(2i/d) with base = theta while that length is at most
// max_pos, else theta * (factor * length / max_pos - (factor - 1))^(d / (d - 2))
int pta_rope_dynamic_table(float* out, const int* seq_start, const int* cu_tokens, int n_seqs, int d, float theta,
                           float factor, int max_pos, void* stream);

// y[M, N] = act(sum of part[P, M, N] over P, in order, + bias) + add1 + add2: the reduction of the products above
// on its own, for 32-bit partial sums over ranges of K that the vendor library's batched product made
int pta_gemm_reduce_parts(void* y, const float* part, const float* bias, const void* add1, const void* add2, int M,
                          int N, int P, int act, int out_f32, void* stream);
// fixes the ranges of K (1..16 each, as pta_gemm_splitk_pair_parts then reports them) for every later pair launch
// of this shape; 0, 0 returns the shape to the built-in rule; returns 1 for counts the kernel does not take
int pta_gemm_splitk_pair_fix_parts(int N1, int K1, int N2, int K2, int p1, int p2);
// the same, and how many tiles of sixteen rows of W a wave holds in steps of more than 32 rows (rt 1 or 2, i.e. 64
// or 128 rows of W a workgroup); the ranges decide the order of summation, the tile height does not
int pta_gemm_splitk_pair_fix(int N1, int K1, int N2, int K2, int p1, int p2, int rt);
// The same two partial products for 1 to 128 rows with the activations stationary (gemm_stationary_bf16.hip):
// about one workgroup per compute unit, each wave keeping the sums of its row tiles in registers while the
// workgroup walks its range of K in phases of LDS-resident slices of x.  parts1 and parts2 ranges of K
// (part1 [parts1, M, N1], part2 [parts2, M, N2], ranges of whole 64-element blocks as in the launches above).
int pta_gemm_stationary_groups(int N1, int K1, int parts1, int N2, int K2, int parts2, int M, int* g1, int* g2);
int pta_gemm_stationary_pair_bf16(float* part1, const void* x1, const void* W1, int N1, int K1, int parts1, float* part2,
                                  const void* x2, const void* W2, int N2, int K2, int parts2, int M, void* stream);
// The pair launch with stationary activations has ranges of K of its own per class of rows (0: up to 16 rows, 1:
// 32, 2: 64, 3: 128): pta_gemm_stationary_rule gives the rule's, pta_gemm_splitk_pair_fix_stationary fixes them for
// a shape and class (0, 0: the staged kernel for that class; cls = -1 forgets the shape; returns 1 for invalid counts).
int pta_gemm_splitk_pair_fix_stationary(int N1, int K1, int N2, int K2, int cls, int q1, int q2);
int pta_gemm_stationary_rule(int N1, int K1, int N2, int K2, int cls, int* q1, int* q2);
int pta_gemm_splitk_pair_bf16(float* part1, const void* x1, const void* W1, int N1, int K1, float* part2,
                              const void* x2, const void* W2, int N2, int K2, int M, void* stream);

// the same pair run to the end: y1 = act1(x1 . W1^T + bias1), y2 = act2(x2 . W2^T + bias2), bfloat16
int pta_gemm_splitk_pair_reduced_bf16(void* y1, float* part1, const void* x1, const void* W1, const float* bias1, int N1,
                                      int K1, int act1, void* y2, float* part2, const void* x2, const void* W2,
                                      const float* bias2, int N2, int K2, int act2, int M, void* stream);

// pta_gemm_splitk_bf16 (rt, parts, stage_blocks, depth chosen, reduce = 1) for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid it.  It has no counterpart in
// the reference.  The partial sums lie in an array that the library holds on every GPU it runs on until the
// process ends (pta_gemm_splitk_static_floats() 32-bit values, 16 MiB); a product whose ranges x M x N exceed that
// is refused with a message.  The call allocates and frees nothing.  All calls on one GPU share that GPU's array,
// which keeps the last call's contents (nothing in it has to start at zero: a call writes every partial sum
// before it reads it): calls that overlap on one GPU (two streams, two threads) race and must be ordered by the
// caller.
int pta_gemm_splitk_bf16_static(void* y, const void* x, const void* W, const float* bias, const void* add1,
                                const void* add2, int M, int N, int K, int act, int out_f32, void* stream);
long pta_gemm_splitk_static_floats(void);

// processors in the reference's order, then argmax (do_sample 0) or a draw; `work` [R, V] is scratch and,
// with want_scores, receives the processed scores (without, its contents are unspecified);
// typical_p 1, epsilon_cutoff 0 and eta_cutoff 0 switch those off; hist/hist_off (tokens seen, per row),
// ban/ban_off (tokens a row may not take, per row), eos/suppress, uniforms may be null.  bias_tok/bias_val/bias_off
// (per row: tokens, each once, whose score gets a value added before anything else; null: none), forced/n_forced
// (in this step every score goes but those of these tokens, which become 0; 0: nothing is forced), decay_on/decay_m
// (the EOS tokens' scores gain |score| * decay_m after the removal of invalid values)
int pta_sample(int* out_tok, float* work, const float* logits, int R, int V, int do_sample, float temperature,
               int top_k, float top_p, float min_p, float typical_p, float epsilon_cutoff, float eta_cutoff,
               float penalty, const int* hist, const int* hist_off, const int* ban, const int* ban_off,
               const int* eos, int n_eos, const int* suppress, int remove_invalid, int renorm, uint64_t seed,
               const int* rng_seq, const int* rng_step, const float* uniforms, int want_scores, const int* bias_tok,
               const float* bias_val, const int* bias_off, const int* forced, int n_forced, int decay_on, float decay_m,
               void* stream);

// out_tok[r] = index of the largest of logits[r, :], lowest index among equals (greedy choice, no processors)
int pta_argmax(int* out_tok, const float* logits, int R, int V, void* stream);

// host function: the uniform number in [0, 1) that pta_sample draws for (seed, sequence, step)
float pta_philox_uniform(uint64_t seed, uint32_t seq, uint32_t step);

#ifdef __cplusplus
}
#endif
