/*
 * katz_hip -- C ABI of the MI355X (gfx950) kernels for the adapter-augmented SDXL UNet hot path.
 *
 * The reference binds its native ops through TORCH_LIBRARY(fast_kernel)
 * (diffusers-hf/src/fast_kernel/fast_kernel/csrc/main.cpp:10-12, bind.cu:12-15) with torch::Tensor
 * signatures; this library is the layer underneath such a binding: plain device pointers, sizes and a
 * stream, no torch types, so it can be bound from torch (ctypes / TORCH_LIBRARY), from C++ or from a
 * standalone benchmark.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; bf16 tensors are raw 16-bit storage;
 *   - tensors are dense row-major unless strides are explicit arguments;
 *   - `stream` is a hipStream_t (NULL = default stream); every call only enqueues work, never
 *     synchronises, never allocates, and is safe under HIP graph capture;
 *   - return value: 0 = enqueued; < 0 = argument rejected before any launch (KH_ERR_*);
 *     > 0 = the hipError_t reported by the launch.  The reference's GroupNorm swallows launch errors
 *     (csrc/group_norm.cu:167-169, :219-221); this ABI never does.
 */
#ifndef KATZ_HIP_H
#define KATZ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KH_OK 0
#define KH_ERR_INVALID_ARG (-1) /* null pointer, non-positive size, inconsistent shape */
#define KH_ERR_UNSUPPORTED (-2) /* shape outside what the kernels are built for (e.g. head_dim != 64) */
#define KH_ERR_ALIGNMENT (-3)   /* a pointer or stride is not 16-byte aligned */
#define KH_ERR_TOO_LARGE (-4)   /* size beyond a documented maximum */

/* ABI version, bumped on any signature change. */
int kh_version(void);
/* Static string for a KH_ERR_* code or a hipError_t (host pointer, never NULL). */
const char* kh_error_string(int code);

/* Per-launch timing for benchmarks (no counterpart in the reference, which times whole steps with
 * torch.cuda.synchronize + time.time, pipeline_controlnet_sd_xl_katz.py:1588-1644).  Between
 * kh_profile_begin and kh_profile_end every kernel of this library is launched with its own HIP
 * start/stop event pair on the launch stream.  kh_profile_end waits for them and writes, in launch
 * order, a kernel tag (1 lora_gemm, 2 lora_gemm_f32, 3 attention, 4 group_norm stats, 5 group_norm apply,
 * 6 layer_norm, 7 geglu, 8 residual_add, 9 concat_residual, 10 sgmv_shrink, 11 sgmv_expand, 12 lora_shrink, 13 conv3x3, 14 cfg_euler, 15 upsample, 16 lora_merge, 17 conv_out + guidance + Euler) and the
 * duration in ms into HOST arrays; returns the number of launches (or -hipError_t).  Do not use under
 * graph capture. */
int kh_profile_begin(void);
int kh_profile_end(int32_t* tags, float* ms, int capacity);

/* ---- K1: LoRA-patched Linear ------------------------------------------------------------------
 * y[M,N] = x[M,K] W[N,K]^T + bias[N] + ((x A_cat[R,K]^T) * col_scale[R]) B_cat[N,R]^T (+ residual[M,N])
 * Replaces base Linear + per-adapter low-rank branch of the reference:
 *   LoRACompatibleLinear.forward  diffusers-hf/src/diffusers/models/lora.py:451-457
 *   LoRALinearLayer.forward       diffusers-hf/src/diffusers/models/lora.py:222-232
 * (the peft Linear injected at diffusers-hf/src/diffusers/loaders/lora.py:409,475-476 computes the same
 * sum over active adapters).  A_cat/B_cat: active adapters concatenated along the rank axis and padded
 * with zero rows/columns to R % 32 == 0, R <= 128; col_scale[r] = weight_i * alpha_i / rank_i of the
 * adapter that owns rank column r (what scale_lora_layers / set_adapters compute on the host,
 * diffusers-hf/src/diffusers/utils/peft_utils.py:103-147,238-269).  R == 0 is a plain Linear.
 * bias, residual may be NULL.  K % 8 == 0, N % 8 == 0.
 * flags bit 0: GEGLU epilogue -- W/bias/B_cat rows are permuted so that every 64 consecutive rows are
 *   32 value rows followed by their 32 gate rows; y is [M, N/2] = value * gelu_erf(gate)
 *   (GEGLU.forward, diffusers-hf/src/diffusers/models/activations.py:139-149); N % 64 == 0, no residual.
 * flags bits 8..15: tile override for tuning (0 = automatic).  Every other bit must be zero (KH_ERR_INVALID_ARG);
 * in particular the r_used promise of the sibling entry points below (bits 16..23) has no meaning here. */
int kh_lora_linear_bf16(const void* x, const void* w, const void* bias, const void* a_cat, const void* b_cat,
                        const float* col_scale, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                        int64_t R, int flags, void* stream);
/* The same layer in two launches, for inputs whose rank-R product is better computed once than once per
 * output tile (and for several layers sharing one input, e.g. to_q/to_k/to_v: stack their A matrices):
 *   kh_lora_shrink_bf16:      t[M,R] = bf16((x[M,K] A_cat[R,K]^T) * col_scale[R])      K % 64 == 0, R % 32 == 0
 *   kh_lora_linear_pre_bf16:  y = x W^T + bias + t[:, 0:R] B_cat[N,R]^T (+ residual | GEGLU)
 * t is [M, ldt] with ldt >= R (a column slice of a wider shrink result is addressed by offsetting the
 * pointer); it is ~1 MB and stays in L2 between the two launches.  Same reference formula as above
 * (lora.py:222-232: up(down(x)) * scale).  K % 32 == 0, R <= 128, flags as for kh_lora_linear_bf16.
 * n_split > 0 fuses several layers with one input into one GEMM (to_q/to_k/to_v): W, bias, B_cat are the
 * layers stacked along N in blocks of n_split rows (n_split % 128 == 0) and block j takes T columns
 * [j*R, (j+1)*R) of the shared shrink result; 0 = a single layer.
 * flags bits 16..23 (kh_lora_linear_pre_bf16, kh_lora_linear_split_bf16): r_used / 16, a promise that the rank columns
 * >= r_used of every layer's t block and B_cat are all zero (the padding of R = sum of the adapters' ranks up to a
 * multiple of 64); the kernels then skip products that could only add zeros.  0 = no promise. */
int kh_lora_shrink_bf16(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M, int64_t K,
                        int64_t R, void* stream);
int kh_lora_linear_pre_bf16(const void* x, const void* w, const void* bias, const void* t, int64_t ldt,
                            int64_t n_split, const void* b_cat, const void* residual, void* y, int64_t M, int64_t N,
                            int64_t K, int64_t R, int flags, void* stream);
/* The two-launch form from its unshrunk operands: y = x W^T + b + ((x A_cat^T) * col_scale) B_cat^T (+ residual | GEGLU)
 * with t_scratch [M,R] bf16 receiving the shrink result (LoRACompatibleLinear.forward, diffusers-hf/src/diffusers/
 * models/lora.py:224-225 + :423-431, as kh_lora_shrink_bf16 followed by kh_lora_linear_pre_bf16).  Where the base
 * GEMM's 128x128 tiles leave at least a quarter of the CUs idle (N = 1280 at M = 2048) the shrink runs INSIDE the GEMM
 * launch on those CUs: its workgroups come first in the grid, store t_scratch write-through and count themselves into
 * `counters`; the GEMM workgroups read t_scratch (as the last K tiles) only after their row block's count is complete.
 * Same results as the two launches up to the fp32 summation order of the shrink.
 * counters: KH_SPLIT_COUNTER_INTS(M) int32 of device memory owned by the caller, ZERO when the call is enqueued;
 * the launch leaves its arrival counts in them, so the caller clears them (a fill kernel; in a HIP graph, one fill
 * over all call sites' counters at the start of the step) before the same memory serves another call.  NULL = always
 * two launches.  The last of them becomes 1 if a bounded wait inside the launch ever ran out (the result of that
 * call is then undefined).  n_split > 0: w / bias / b_cat stack N / n_split layers of n_split rows each (q, k, v of a
 * self-attention), a_cat / col_scale stack their A matrices ([N / n_split * R, K]) and t_scratch is [M, N / n_split * R],
 * as for kh_lora_linear_pre_bf16.  K % 64 == 0, R % 32 == 0, R <= 128.  flags: bit 0 GEGLU, bits 8..15: 1 = always two
 * launches, bits 16..23: r_used / 16 as above, bit 24: never the cooperative form (below).
 * Cooperative form: where the GEMM's 128x160 tiles give every CU exactly one workgroup (N = 640 at M = 8192), R = 128 and
 * 0 < r_used <= 96, no CU is idle, and EVERY workgroup first computes a 32-row x 96-column piece of its row block's
 * t_scratch, counts itself into `counters` and only then runs its tile, waiting (bounded, as above) for the four pieces
 * of its row block before the last K tiles.  No workgroup waits before its own piece is out, so one such launch always
 * completes; TWO of them running at the same time on different streams can each hold the CUs the other's not yet
 * started workgroups need, and then both only end through the bounded wait.  A caller that enqueues these calls on
 * streams that may overlap sets bit 24 on all but one of the streams. */
#define KH_SPLIT_COUNTER_INTS(M) (((M) + 127) / 128 + 1)
int kh_lora_linear_split_bf16(const void* x, const void* w, const void* bias, const void* a_cat, const float* col_scale,
                              const void* b_cat, void* t_scratch, int32_t* counters, const void* residual, void* y,
                              int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split, int flags, void* stream);
/* The LoRA linear of kh_lora_linear_split_bf16 with the LayerNorm in front of it folded into the GEMM, and / or with the
 * row statistics a folded LayerNorm BEHIND it needs written by its epilogue.  The reference's transformer block runs
 * norm -> projection three times (diffusers-hf/src/diffusers/models/attention.py:338-403: norm1 -> attn1.to_q/k/v,
 * norm2 -> attn2.to_q, norm3 -> ff.net.0.proj), each norm a pass over the hidden states of its own; here the producer
 * of the hidden states (attn.to_out.0 / ff.net.2 / proj_in with their residual) leaves per-row partial sums, and the
 * consumer GEMM reads the UN-normalised rows and finishes the normalisation per output element:
 *   LN(x) W^T + b  =  rstd_m * (x W'^T - mean_m * c1) + c2,   W' = W * gamma (per K column),
 *                     c1[n] = sum_k W'[n,k],  c2[n] = b[n] + sum_k beta[k] W[n,k].
 * stats_out (may be NULL): float [16][M][2]; column tile j of the GEMM writes (sum, sum of squares) of its columns of
 *   every output row (after bias and residual, over the bf16-rounded values) to pair [j][row], the pairs past the
 *   last tile are zeroed.  N <= 2048, no GEGLU.
 * ln_part (may be NULL): such an array for the rows of x.  Then w must be W' (and a_cat must be A_cat * gamma), bias
 *   must be NULL (it is part of ln_c2), ln_c1 / ln_c2 are float [N] as above and, with R > 0, ln_ca1[r] = sum_k
 *   a_cat'[r,k], ln_ca2[r] = sum_k beta[k] A_cat[r,k] (float [rows of a_cat]) let the shrink store
 *   ((x A'^T) - mean * ca1 + ca2 / rstd) * col_scale, the adapters' share before the common factor rstd.
 *   mean = sum / K, rstd = rsqrt(sumsq / K - mean^2 + ln_eps): the formula of kh_layer_norm_bf16.
 * R == 0: plain linear (a_cat, col_scale, b_cat, t_scratch, counters NULL).  Everything else (counters, n_split, flags,
 * shape limits) as for kh_lora_linear_split_bf16.  Results differ from LayerNorm followed by the linear by rounding
 * only: the normalised row is never rounded to bf16, W' is. */
int kh_lora_linear_norm_bf16(const void* x, const void* w, const void* bias, const void* a_cat, const float* col_scale,
                             const void* b_cat, void* t_scratch, int32_t* counters, const void* residual, void* y,
                             const float* ln_part, const float* ln_c1, const float* ln_c2, const float* ln_ca1,
                             const float* ln_ca2, float ln_eps, float* stats_out, int64_t M, int64_t N, int64_t K,
                             int64_t R, int64_t n_split, int flags, void* stream);
/* A cross-attention's query projection and the attention itself in ONE launch: o = softmax(q k^T * scale) v with
 * q = kh_lora_linear_norm_bf16(x, ...) never written to memory.  The reference runs to_q, then the attention processor
 * on its result (diffusers-hf/src/diffusers/models/attention_processor.py:1231-1296: attn.to_q :1256, head split
 * :1269-1272, F.scaled_dot_product_attention :1276); on the SDXL text context (S = 77 keys) the attention alone is a
 * launch of a few microseconds whose 128 queries x 2 heads are exactly one 128 x 128 output tile of the projection, so
 * the GEMM's epilogue keeps the tile in LDS, loads the S keys / values of its two heads and runs the attention there.
 * x [M,K] with M = B * T (rows of sample b: b*T .. b*T + T - 1), w [N,K], N = heads * 64; k, v: [B,S,N] views (row
 * strides ldk / ldv, sample strides bsk / bsv, in elements); o [M,N] with row stride ldo, head h at columns 64 h.
 * The projection's arguments (bias, adapters, t_scratch, counters, folded LayerNorm, flags bits 8..23) are
 * kh_lora_linear_norm_bf16's, without residual, statistics, GEGLU and n_split.  M % 128 == 0, T % 128 == 0, N % 128 == 0,
 * K % 64 == 0, R % 64 == 0, R <= 128, S <= 96, at most 256 tiles of 128 x 128: kh_lora_linear_xattn_ok says whether a
 * shape is taken (1) or not (0: run the projection and kh_attention_bf16).  Against those two calls the result differs
 * by rounding only (one softmax pass over all keys instead of a running maximum over 64-key tiles). */
int kh_lora_linear_xattn_bf16(const void* x, const void* w, const void* bias, const void* a_cat, const float* col_scale,
                              const void* b_cat, void* t_scratch, int32_t* counters, const float* ln_part,
                              const float* ln_c1, const float* ln_c2, const float* ln_ca1, const float* ln_ca2, float ln_eps,
                              const void* k, const void* v, void* o, int64_t M, int64_t N, int64_t K, int64_t R, int64_t T,
                              int64_t S, int64_t ldk, int64_t ldv, int64_t ldo, int64_t bsk, int64_t bsv, float scale,
                              int flags, void* stream);
int kh_lora_linear_xattn_ok(int64_t M, int64_t N, int64_t K, int64_t R, int64_t T, int64_t S);
/* Bounded waits of kh_lora_linear_split_bf16's in-launch shrink that have run out on the current device since the
 * process started (or since the last call with clear != 0): writes the number to *count (HOST pointer).  A GEMM workgroup
 * of that launch waits for the shrink workgroups of the same launch, which have lower workgroup ids and are therefore
 * dispatched first (in the cooperative form: for the other workgroups of its row block, each of which delivers its piece
 * before it waits); the wait gives up after 2^20 polls (about a quarter of a second) and the result of that call is then
 * undefined.  The flag word in `counters` says so per call but is wiped by the caller's next reset; this count is not.
 * A non-zero value means results since the last check cannot be trusted.  Blocks until the device's earlier work is
 * done (a 4-byte copy on the null stream); not under graph capture.  No counterpart in the reference. */
int kh_lora_split_timeouts(int32_t* count, int clear);
/* Weight prefetch hint; no counterpart in the reference (its cuBLAS / cuDNN calls take no such hint).  The next launch of
 * the linear / convolution family made by this host thread (kh_lora_linear_bf16, _pre, _split, _norm, kh_conv3x3_nhwc_bf16)
 * also touches every 128-byte line of weights[0 .. bytes): an operand of the launch that FOLLOWS it, so that it is in
 * the memory-side cache when that launch asks for it.  Up to three ranges may be queued by consecutive calls (weights,
 * A_cat, B_cat; of the second and third at most the first 16 MB are touched); a fourth returns KH_ERR_TOO_LARGE.
 * A UNet step reads its 2.5 GB of weights once each, so every launch would otherwise meet its weights in HBM, and each
 * XCD that shares a weight block would fetch it again; measured on the SDXL feed-forward output projection (M 2048,
 * N 1280, K 5120): 53 us with the weights in HBM, 45 us prefetched, 42 us cache-resident.  The hints are consumed by
 * that one launch (also under graph capture, where the pointers are recorded: the ranges must stay allocated while the
 * graph is replayed).  A call of that family drops whatever is pending when it returns, also when it refuses its
 * arguments before launching: a hint never survives to a later, unrelated launch.  weights == NULL or bytes < 128
 * clears what is pending.  At most 2 GiB per range.  Wrong hints cost bandwidth, never correctness; the ranges must be
 * readable.  The Python host issues hints only inside one forward of one model and only at that model's own tensors
 * (katz_amd/ops.py weight_prefetch_scope), so a captured graph of a model records hinted pointers into that model only. */
int kh_set_weight_prefetch(const void* weights, int64_t bytes);
/* How many kernel launches kh_lora_linear_split_bf16 makes for this shape when counters are given (1 or 2; negative:
 * KH_ERR_*).  No counterpart in the reference; for callers that account per launch (benchmarks). */
int kh_lora_linear_split_launches(int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split, int flags);
/* n_groups layers that read the SAME x in one launch (the context K/V projections of every cross-attention
 * of the UNet: 140 GEMMs of 154 rows each, which individually cannot fill the chip):
 *   y_g = x W_g^T + bias_g + t_g B_cat_g^T        g = 0 .. n_groups-1, all with the same M, N, K, R
 * table: DEVICE array of n_groups rows of five 64-bit device addresses {W_g, bias_g or 0, B_cat_g or 0,
 * t_g or 0, y_g}; t_g addresses a [M, ldt] matrix (typically a column slice of one wide shrink result).
 * R == 0: plain linears.  No counterpart in the reference (it issues the layers one by one,
 * attention_processor.py:1260-1262).  K % 32 == 0, R <= 128, no GEGLU / residual. */
int kh_lora_linear_grouped_bf16(const void* x, const uint64_t* table, int64_t n_groups, int64_t ldt, int64_t M,
                                int64_t N, int64_t K, int64_t R, int flags, void* stream);
/* Merge adapters into the weights of MANY layers in one launch:  W_l += scale * layer_scale[l] * up_l . down_l.
 * Replaces the per-layer loop of Katz's patch_on_lora, `unet_state_dict[key] += cur_up @ cur_down * scale`
 * (diffusers-hf/src/diffusers/pipelines/controlnet/pipeline_controlnet_sd_xl_katz.py:1737-1747), and the per-module
 * _fuse_lora of diffusers-hf/src/diffusers/models/lora.py:403-433; the product is accumulated in fp32 and the sum
 * rounded once.  table: DEVICE array of n_layers rows of six 64-bit words {W, up, down, N, K, r}: device addresses of
 * W [N,K] (bf16, updated in place), up [N,r], down [r,K], then the three sizes as int64.  up / down are bf16 storage,
 * or float16 when operands_fp16 != 0 (the dtype of Katz's shared-memory adapter arrays, load_lora_shm_multi.py:49-61).
 * tile_start: DEVICE int32 [n_layers + 1], tile_start[l] = sum over layers before l of ceil(N/128) * ceil(K/128);
 * total_tiles = tile_start[n_layers] (sizes the grid).  layer_scale: DEVICE float [n_layers] or NULL (all 1).
 * max_rank: the largest r in the table (<= 128; sizes the kernel's LDS).  A negative scale undoes a merge up to
 * rounding.  The same W must not appear in two rows. */
int kh_lora_merge_grouped_bf16(const uint64_t* table, const int32_t* tile_start, const float* layer_scale,
                               int64_t n_layers, int64_t total_tiles, int64_t max_rank, float scale, int operands_fp16,
                               void* stream);
/* fp32 variant of the same formula (fp32 parity path); R <= 128, any M/N/K. */
int kh_lora_linear_f32(const float* x, const float* w, const float* bias, const float* a_cat, const float* b_cat,
                       const float* col_scale, const float* residual, float* y, int64_t M, int64_t N, int64_t K,
                       int64_t R, void* stream);

/* ---- K2: segmented multi-adapter shrink / expand ----------------------------------------------
 * Per-request adapters in one batch: segment s = rows [seg_start[s], seg_start[s+1]) uses adapter
 * seg_adapter[s] (< 0: none).  No counterpart in the reference; semantics = the LoRA linear above
 * applied request by request (lora.py:222-232).  a_all [n_adapters, RP, K], b_all [n_adapters, N, RP],
 * t [rows_total, RP]; adapter_rank[a] = rank rounded up to a multiple of 32 (zero padded), RP <= 128.
 * seg_start (n_segments+1), seg_adapter, adapter_rank: device int32; adapter_scale: device float.
 * max_seg_rows = longest segment (sizes the grid).
 *   shrink: t[rows, 0:r] = x[rows,:] A_a^T          expand: y[rows,:] += scale_a * t[rows,0:r] B_a^T
 * with r = adapter_rank[a]; the shrink leaves the columns t[rows, r:RP] as they were (the expand never reads them). */
int kh_sgmv_shrink_bf16(const void* x, const void* a_all, void* t, const int32_t* seg_start,
                        const int32_t* seg_adapter, const int32_t* adapter_rank, int64_t n_segments,
                        int64_t max_seg_rows, int64_t K, int64_t RP, void* stream);
int kh_sgmv_expand_bf16(const void* t, const void* b_all, void* y, const int32_t* seg_start,
                        const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                        int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t RP, void* stream);
/* Both in one launch: y[rows,:] += scale_a * bf16(x[rows,:] A_a^T) B_a^T per segment, t kept inside the workgroup (no
 * counterpart in the reference, as above; the arithmetic and roundings of kh_sgmv_shrink_bf16 followed by
 * kh_sgmv_expand_bf16).  K % 64 == 0, N % 128 == 0, RP % 32 == 0, RP <= 128; other shapes: KH_ERR_UNSUPPORTED (use the
 * two launches). */
int kh_sgmv_fused_bf16(const void* x, const void* a_all, const void* b_all, void* y, const int32_t* seg_start,
                       const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                       int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t K, int64_t RP, void* stream);
/* The same for n_layers layers that read the SAME x with the SAME segments (the to_k / to_v projections of all
 * cross-attentions of one width read the one text context, diffusers-hf/src/diffusers/models/attention_processor.py:1246-1251)
 * in one launch: table = n_layers rows of three device pointers {a_all_l, b_all_l, y_l} (8-byte aligned device memory; the
 * pointed-to arrays as in kh_sgmv_fused_bf16, 16-byte aligned, all layers with the same N, K, RP and adapter table).
 * A 77-row request gives one layer's launch a few microseconds of traffic; all layers of a width together are bound by
 * the memory system instead of by the launch.  No counterpart in the reference. */
int kh_sgmv_fused_grouped_bf16(const void* x, const uint64_t* table, int64_t n_layers, const int32_t* seg_start,
                               const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                               int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t K, int64_t RP, void* stream);

/* ---- K3: attention ----------------------------------------------------------------------------
 * o = softmax(q k^T * scale) v per (batch, head); replaces F.scaled_dot_product_attention in
 * AttnProcessor2_0.__call__ (diffusers-hf/src/diffusers/models/attention_processor.py:1269-1283).
 * q,o: [B,T,H*64]; k,v: [B,S,H*64] addressed with row strides ld* and batch strides bs* (elements,
 * multiples of 8), so q/k/v may be column slices of a fused projection.  head_dim must be 64. */
int kh_attention_bf16(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t T,
                      int64_t S, int64_t head_dim, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t bsq,
                      int64_t bsk, int64_t bsv, int64_t bso, float scale, void* stream);

/* ---- K4: GroupNorm (+SiLU), LayerNorm -----------------------------------------------------------
 * Replaces torch.ops.fast_kernel.group_norm_fp16(x, y, eps, num_groups, activation, weight, bias,
 * affine, channels_last) (csrc/group_norm.cu:264-274, called at
 * diffusers-hf/src/diffusers/models/normalization.py:90-91); y is caller-allocated as there.
 * activation: 0 none, 1 silu.  channels_last: 1 = x,y are [N,HW,C] (NHWC), 0 = [N,C,HW] (NCHW).
 * gamma/beta may be NULL (affine=False).  add_nc (may be NULL): bf16 [N,C] added to x per (sample,
 * channel) before the statistics and the normalisation -- folds the resnet's `hidden_states + temb`
 * (diffusers-hf/src/diffusers/models/resnet.py:388-390) into the norm that follows it.  workspace: kh_group_norm_workspace_bytes(...) bytes of
 * device memory owned by the caller (the reference allocates its mean/inv_variance tensors per call,
 * group_norm.cu:240-242, which is not graph-capturable).  NHWC needs C % 8 == 0, C <= 4096, G <= 512;
 * NCHW needs HW % 8 == 0. */
int64_t kh_group_norm_workspace_bytes(int64_t N, int64_t C, int64_t HW, int64_t G, int channels_last);
int kh_group_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                       float* workspace, int64_t N, int64_t C, int64_t HW, int64_t G, float eps, int activation,
                       int channels_last, void* stream);
/* The second pass of kh_group_norm_bf16 alone (channels_last only), on statistics another kernel has left:
 * partials float [N * G * splits * 2], (sum, sum of squares) of x + add_nc per (sample, group, split) in any split of the
 * sample's pixels (kh_conv3x3_gn_stats_nhwc_bf16 writes them).  Folds them in fp64 in a fixed order and writes
 * y = act((x + add_nc - mean) * rstd * gamma + beta).  Arguments otherwise as for kh_group_norm_bf16. */
int kh_group_norm_apply_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                             const float* partials, int64_t splits, int64_t N, int64_t C, int64_t HW, int64_t G, float eps,
                             int activation, void* stream);
/* kh_group_norm_bf16 for callers that cannot allocate device memory (code under HIP graph capture whose allocator is
 * out of reach, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference (its op
 * allocates two tensors per call, group_norm.cu:240-242).  Same arguments without `workspace`; same kernels, same
 * results bit for bit.  The partial statistics go to a 256 KiB array that the library holds in the memory of every GPU
 * it runs on until the process ends; shapes whose kh_group_norm_workspace_bytes(...) exceeds 256 KiB (none of the
 * SDXL UNet / ControlNet norms: they need <= 33 KiB) return KH_ERR_TOO_LARGE.  The call allocates nothing.  All calls
 * on one GPU share the array: calls that can overlap on one GPU (different streams, several host threads) race; calls
 * on one stream are ordered.  The first call on a device looks up the array's address (no allocation, no launch);
 * make that call outside graph capture. */
int kh_group_norm_static_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                              int64_t N, int64_t C, int64_t HW, int64_t G, float eps, int activation,
                              int channels_last, void* stream);
/* nn.LayerNorm over the last axis (norm1/2/3 of BasicTransformerBlock,
 * diffusers-hf/src/diffusers/models/attention.py:195,225,253); D % 8 == 0, D <= 2048. */
int kh_layer_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, int64_t M, int64_t D, float eps,
                       void* stream);

/* ---- K5: GEGLU -----------------------------------------------------------------------------------
 * out[M,D] = proj[M, 0:D] * gelu(proj[M, D:2D])  (GEGLU.forward unfused branch, activations.py:148-149;
 * approximate_tanh = 0 is F.gelu's exact erf form, 1 the tanh form of csrc/gelu.cuh:29-42). */
int kh_geglu_bf16(const void* proj, void* out, int64_t M, int64_t D, int approximate_tanh, void* stream);
/* out = gelu(x) * m, n elements: torch.ops.fast_kernel.fast_gelu_mul_fp16(x, m)
 * (csrc/gelu.cuh:44-59, called at activations.py:145); the caller allocates out. */
int kh_gelu_mul_bf16(const void* x, const void* m, void* out, int64_t n, int approximate_tanh, void* stream);

/* ---- ControlNet residual injection -----------------------------------------------------------------
 * dst[n] += (sum_k srcs[k][n]) * inv_count : skip_j + r_j and sample + r_mid
 * (diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1284-1292), with the multi-ControlNet
 * sum then mean of :1418-1439 folded in (inv_count = 1/#ControlNets).  srcs: HOST array of n_srcs (<= 8)
 * device pointers; n % 8 == 0. */
int kh_residual_add_bf16(void* dst, const void* const* srcs, int n_srcs, float inv_count, int64_t n, void* stream);
/* Channels-last concat with the residual add folded in:
 * out[rows, 0:C1] = h[rows, C1]; out[rows, C1:C1+C2] = skip[rows, C2] + (sum_k residuals[k]) * inv_count.
 * Replaces torch.cat([hidden_states, res_hidden_states], dim=1) of the up blocks
 * (diffusers-hf/src/diffusers/models/unets/unet_2d_blocks.py:2512, :2645) plus the adds above.
 * residuals: HOST array of n_residuals (0..8) device pointers; C1 % 8 == 0, C2 % 8 == 0. */
int kh_concat_residual_bf16(const void* h, const void* skip, const void* const* residuals, int n_residuals,
                            float inv_count, void* out, int64_t rows, int64_t C1, int64_t C2, void* stream);
/* Nearest-neighbour 2x upsampling of an NHWC tensor: y[n, h, w, :] = x[n, h/2, w/2, :], y is [N, 2H, 2W, C].
 * Replaces F.interpolate(hidden_states, scale_factor=2.0, mode="nearest") of Upsample2D.forward
 * (diffusers-hf/src/diffusers/models/upsampling.py:169-171) in front of the upsampler's convolution.  C % 8 == 0. */
int kh_upsample_nearest2x_nhwc_bf16(const void* x, void* y, int64_t N, int64_t H, int64_t W, int64_t C, void* stream);

/* ---- 3x3 convolution of the residual blocks ------------------------------------------------------------
 * y[n,ho,wo,co] = bias[co] + sum_{kh,kw,ci} x[n, ho*stride+kh-1, wo*stride+kw-1, ci] * w[co,kh,kw,ci]
 *                 (+ residual[n,ho,wo,co]); zero padding 1, stride 1 or 2, Ho = (H-1)/stride + 1.
 * conv1 / conv2 of ResnetBlock2D (diffusers-hf/src/diffusers/models/resnet.py:275, :295, applied at :351, :369),
 * the stride-2 conv of Downsample2D and the conv of Upsample2D (diffusers-hf/src/diffusers/models/downsampling.py,
 * upsampling.py), with the block's `input_tensor + hidden_states` (resnet.py:374) as the optional residual.
 * Layout: x NHWC [Nb,H,W,Cin], w [Cout,3,3,Cin] (the nn.Conv2d weight permuted to O,KH,KW,I), y and residual
 * NHWC [Nb,Ho,Wo,Cout], all bf16; bias bf16 [Cout] or NULL.  Runs as an implicit GEMM (M = Nb*Ho*Wo,
 * K = 9*Cin) on the MFMA pipeline of kh_lora_linear_bf16.  Cin % 32 == 0, Cout % 8 == 0. */
int kh_conv3x3_nhwc_bf16(const void* x, const void* w, const void* bias, const void* residual, void* y, int64_t Nb,
                         int64_t H, int64_t W, int64_t Cin, int64_t Cout, int64_t stride, void* stream);
/* A convolution of a residual block that leaves the statistics of the GroupNorm behind it as a by-product of its epilogue:
 *   y = conv3x3(x) + bias (+ residual), exactly as kh_conv3x3_nhwc_bf16, and per (image, group, row tile of the image) the
 *   (sum, sum of squares) of y + add_nc[n, c] over the tile's pixels and the group's channels
 * -- conv1, `hidden_states + temb`, then norm2 of ResnetBlock2D.forward (diffusers-hf/src/diffusers/models/resnet.py:378,
 * :389, :390), and conv2 with the block's skip (resnet.py:408-413) in front of the next module's GroupNorm (the
 * transformer's, transformers/transformer_2d.py:481, or the next block's norm1).  fast_kernel's group_norm_fp16 (normalization.py:91)
 * reads the activation twice (statistics, then normalisation); here the first of the two reads never happens: the
 * convolution's output tiles hold whole groups, so their workgroups sum them while the tile is still in LDS, and
 * kh_group_norm_apply_bf16 folds the partial sums (fp64, fixed order) and normalises.  The statistics are taken over the
 * bf16-rounded stored result plus add_nc, as kh_group_norm_bf16 takes them from memory: against convolution +
 * kh_group_norm_bf16 the result differs by the summation order of the statistics only.
 * kh_conv3x3_gn_splits(...) = row tiles per image when the shape is taken (the convolution runs on 160-column tiles,
 * Cout % 160 == 0, 160 % (Cout / G) == 0, whole tiles per image: every resnet convolution of SDXL), else 0 (run
 * kh_conv3x3_nhwc_bf16 and kh_group_norm_bf16).  partials: float [Nb * G * splits * 2], written completely.
 * add_nc bf16 [Nb, Cout] or NULL.  Everything else as for kh_conv3x3_nhwc_bf16. */
int64_t kh_conv3x3_gn_splits(int64_t Nb, int64_t H, int64_t W, int64_t Cin, int64_t Cout, int64_t stride, int64_t G);
int kh_conv3x3_gn_stats_nhwc_bf16(const void* x, const void* w, const void* bias, const void* residual, const void* add_nc,
                                  void* y, float* partials, int64_t Nb, int64_t H, int64_t W, int64_t Cin, int64_t Cout,
                                  int64_t stride, int64_t G, void* stream);

/* ---- Classifier-free guidance + Euler step --------------------------------------------------------------
 * eps = u + g*(t - u) with noise_pred = [u; t] (uncond rows first)      pipeline_controlnet_sd_xl_katz.py:1649-1650
 * x0 = x - sigma*eps; d = (x - x0)/sigma; x' = x + d*(sigma_next - sigma) scheduling_euler_discrete.py:505-527
 *                                                                        (epsilon prediction, s_churn = 0)
 * model_input_next = [x'; x'] / next_scale                               pipeline :1565-1570 + scale_model_input,
 *                                                                        scheduling_euler_discrete.py:274-298
 * in one pass over the latents, fp32 arithmetic in that order.  noise_pred [2,n] bf16; latents / latents_out [n]
 * bf16 (the reference casts prev_sample to the model dtype, :530) or fp32 when latents_f32 != 0; model_input_next
 * [2,n] bf16 or NULL.  coef: DEVICE pointer to {sigma, sigma_next, next_scale = sqrt(sigma_next^2 + 1)} so that a
 * captured graph can be replayed for every step with the three floats rewritten between replays.  n % 8 == 0.
 * latents_out may equal latents (update in place); model_input_next must not overlap noise_pred. */
int kh_cfg_euler_step_bf16(const void* noise_pred, const void* latents, void* latents_out, void* model_input_next,
                           int64_t n, float guidance_scale, const float* coef, int latents_f32, void* stream);

/* The UNet's last convolution with the guidance + Euler step above as its epilogue: the whole tail of a denoising
 * step, from the output of conv_norm_silu to the next step's model input, in one launch.
 *   noise_pred = conv3x3(x, w) + bias          conv_out, unet_2d_condition.py:1327-1331 (4 output channels, padding 1)
 *   then exactly kh_cfg_euler_step_bf16 on noise_pred rounded to bf16 (the model's output dtype).
 * x: NHWC [2*Bl, H, W, Cin] bf16, rows 0..Bl-1 unconditional, Bl..2Bl-1 text-conditioned (the reference's
 * torch.cat([latents] * 2) order, pipeline :1565); w [4,3,3,Cin] (the nn.Conv2d weight permuted to O,KH,KW,I);
 * bias bf16 [4] or NULL; latents / latents_out [Bl,H,W,4] in NHWC memory, bf16 or fp32 (latents_f32), may be the same
 * buffer; model_input_next [2*Bl,H,W,4] bf16 or NULL; noise_pred_out [2*Bl,H,W,4] bf16 or NULL (for callers that
 * want the UNet's output as well); coef as for kh_cfg_euler_step_bf16.  Cin % 16 == 0. */
int kh_conv_out_cfg_euler_bf16(const void* x, const void* w, const void* bias, const void* latents, void* latents_out,
                               void* model_input_next, void* noise_pred_out, int64_t Bl, int64_t H, int64_t W,
                               int64_t Cin, float guidance_scale, const float* coef, int latents_f32, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KATZ_HIP_H */
