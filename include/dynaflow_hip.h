/*
 * dynaflow_hip.h - C ABI of the MI355X (gfx950) kernel library behind the
 * DynaFlow scheduling layer.
 *
 * The reference has no kernel library of its own: its sub-graphs run whatever
 * PyTorch dispatches for their FX nodes (dynaflow/runtime/engine.py:160,220,
 * 325,381,491), optionally compiled by TorchInductor
 * (dynaflow/executor/inductor.py:111-141).  This library takes that slot for
 * the batch-split SwiGLU MLP path.  Each entry point below names the
 * reference call site or kernel whose arithmetic it replaces.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes, no framework types; pointers are device
 *     pointers unless stated otherwise;
 *   - the HIP stream is passed explicitly (NULL = the null stream);
 *   - nothing allocates, frees or synchronises; every call is legal under
 *     stream capture;
 *   - the return value is DFHIP_OK (0) or a negative dfhip_status; shapes,
 *     strides and alignment are checked before anything is launched;
 *   - row-major matrices with leading dimensions given in ELEMENTS;
 *   - bf16 values are the upper 16 bits of an IEEE fp32 (uint16_t storage),
 *     fp8 values are OCP e4m3fn (uint8_t storage).
 */
#ifndef DYNAFLOW_HIP_H
#define DYNAFLOW_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* dfhip_stream_t; /* hipStream_t */

typedef enum dfhip_status {
  DFHIP_OK = 0,
  DFHIP_ERR_NULL_POINTER = -1,
  DFHIP_ERR_BAD_SHAPE = -2,     /* non-positive or unsupported extents */
  DFHIP_ERR_BAD_STRIDE = -3,    /* leading dimension smaller than the row, or of 2^22 (bf16) / 2^23 (fp8)
                                   elements and more for a GEMM operand */
  DFHIP_ERR_BAD_ALIGNMENT = -4, /* pointer or stride not 16-byte aligned */
  DFHIP_ERR_LAUNCH = -5,        /* hipGetLastError() after the launch */
  DFHIP_ERR_NO_DEVICE = -6,
  DFHIP_ERR_BAD_ARGUMENT = -7,
  DFHIP_ERR_TOO_LARGE = -8      /* the problem needs more scratch memory than the library holds */
} dfhip_status;

typedef struct dfhip_device_info {
  int compute_units;
  int clock_khz;           /* peak engine clock */
  int memory_clock_khz;
  int memory_bus_bits;
  int lds_bytes_per_block; /* max opt-in LDS per workgroup */
  int wavefront_size;
  char arch_name[64];      /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
} dfhip_device_info;

/* Library ABI version (major*1000 + minor).  This and the next two have no counterpart in the
 * reference (its sub-graphs call PyTorch, dynaflow/runtime/engine.py:381, which reports its own
 * errors): housekeeping for whoever binds the library. */
int dfhip_version(void);
/* The architecture the device code was compiled for ("gfx950"). */
const char* dfhip_arch(void);
/* Text for a dfhip_status. */
const char* dfhip_status_string(int status);
/* Properties of `device` (host struct).  Counterpart of the cached
 * attribute helpers in
 * examples/ae/scheduler/vllm/tokenweave-kernels/csrc/cuda_utils.cu:3-26. */
int dfhip_device_info_get(int device, dfhip_device_info* out);

/* ------------------------------------------------------------------ GEMMs
 *
 * C[M,N] = A[M,K] * W[N,K]^T  - the `linear` FX node of the sub-graphs
 * (torch.nn.functional.linear, weight stored [out_features, in_features];
 * launched at dynaflow/runtime/engine.py:381).  fp32 accumulation.
 *
 * bf16: A, W, C are bf16.  Requires K % 64 == 0, N % 8 == 0, lda/ldw/ldc % 8
 * == 0 and 16-byte aligned pointers.  Any M >= 1.
 */
int dfhip_gemm_bf16_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                       int64_t ldc, int M, int N, int K, dfhip_stream_t stream);

/* Same contraction (the `linear` node, dynaflow/runtime/engine.py:381) with an explicit kernel
 * variant, for tuning and tests; the choice itself has no counterpart in the reference, where
 * PyTorch picks its GEMM kernel out of sight.
 * variant: 0 = 256x256 tile, LDS-DMA ring (the fast path);
 *          5 = 256x224 tile, LDS-DMA ring (chosen when N = 7 * 2^k makes 224-wide
 *              tiles fill the rounds of 256 workgroups better, e.g. N = 14336);
 *          6 = 128x128 tiles for M <= 1024 (decode-sized activations): W streamed once
 *              through an LDS-DMA ring, K split over workgroups (see _nt_splitk); the
 *              plan picks it up to 128 rows, and up to 512 rows (1024 with K <= 8192)
 *              while the tiles fit one round of 256 workgroups;
 *          7 = 256x128 tile, LDS-DMA ring (chosen instead of a split along K when the
 *              256x256 tiling has few tiles and K <= 8192);
 *          register-staged tiles: 1 = 256x256 / 8 waves, 2 = 128x128 / 4 waves,
 *          3 = 256x128 / 4 waves, 4 = 256x256 / 4 waves. */
int dfhip_gemm_bf16_nt_variant(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                               int64_t ldc, int M, int N, int K, int variant,
                               dfhip_stream_t stream);

/* The kernel choice dfhip_gemm_bf16_nt makes for a shape (variant as above; no counterpart in the
 * reference, see there) and
 * the split_k a caller with a workspace should pass to dfhip_gemm_bf16_nt_splitk
 * (1 = no split). */
int dfhip_gemm_bf16_plan(int M, int N, int K, int* variant, int* split_k);
/* The same choice for a launch that runs side by side with `share` - 1 others of its shape (the same
 * sub-graph of other nano-batches on streams of their own; the scheduler's stream assignment at
 * examples/ae/scheduler/hf/nanoflow.py:122-146 decides that): the launches fill the compute units
 * together, so K is split less or not at all and the tile shape is chosen for the rounds they take
 * together.  1 <= share <= 16; share = 1 is dfhip_gemm_bf16_plan. */
int dfhip_gemm_bf16_plan_shared(int M, int N, int K, int share, int* variant, int* split_k);

/* Split-K flavour of the fast path for shapes with few output tiles (the same `linear` node,
 * dynaflow/runtime/engine.py:381; the down projection of the host model's MLP, whose gate and up
 * projections examples/ae/scheduler/hf/nanoflow.py:30 names: [2048,14336] x [4096,14336]^T has 128 tiles of 256x256 for 256
 * compute units).  Each tile is computed by `split_k` workgroups over disjoint
 * K ranges.  With the 256x256 ring kernel parts 0 .. split_k-2 leave their fp32
 * block in `workspace` and count themselves in; the last part waits for that
 * count, adds the blocks to its own sum in part order (deterministic) and writes
 * C.  The launch is part-major (workgroups [p * tiles, (p + 1) * tiles) are part
 * p of every tile, see dfhip_gemm_bf16_splitk_work), so the part that waits has
 * the highest launch index of its tile for every tile count and whoever it waits
 * for was dispatched before it.  The wait is bounded (about a second); a tile
 * whose parts never arrived is written as NaN.  With the weight-streaming kernel
 * (variant 6) every part leaves a block and the part that arrives last adds them
 * up; nobody waits.  `workspace` (device memory, 16-byte aligned,
 * at least dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k) bytes) starts
 * with the per-tile arrival counters, which must be ZERO before the first use
 * and are left zero by every launch; launches that may overlap in time need
 * workspaces of their own.  1 <= split_k <= 8 (16 where the plan picks the
 * weight-streaming kernel, variant 6), split_k <= K / 64. */
size_t dfhip_gemm_bf16_splitk_workspace_bytes(int M, int N, int split_k);
int dfhip_gemm_bf16_nt_splitk(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                              int64_t ldc, int M, int N, int K, int split_k, void* workspace,
                              size_t workspace_bytes, dfhip_stream_t stream);
/* Host-side replay of the launch order of the 256x256 split-K kernel: which tile and which part of K
 * the workgroup with launch index `launch_index` computes in a launch over `tiles` tiles (launch
 * indices 0 .. tiles * split_k - 1).  Touches no device; it exists so that the ordering argument above
 * (the waiting part is the last of its tile to be dispatched) can be checked on any machine.  No
 * counterpart in the reference. */
int dfhip_gemm_bf16_splitk_work(int launch_index, int tiles, int split_k, int* tile, int* part);

/* dfhip_gemm_bf16_nt_splitk without a workspace argument and without any allocation: the arrival
 * counters and fp32 partial blocks live in a device array of DFHIP_SPLITK_STATIC_BYTES that is part
 * of the library's code object (every GPU the library runs on holds its own copy until the process
 * ends).  It has no counterpart in the reference; it is for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * arguments, checks and result bits as dfhip_gemm_bf16_nt_splitk.  A problem whose
 * dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k) exceeds DFHIP_SPLITK_STATIC_BYTES is refused
 * with DFHIP_ERR_TOO_LARGE (the limit holds the down projection of a 2048-token nano-batch,
 * [2048,14336] x [4096,14336]^T with split_k = 2).  All calls on one GPU share the one array: calls
 * that may overlap in time on a GPU (different streams, different threads) race and must use
 * dfhip_gemm_bf16_nt_splitk with workspaces of their own.  The counters are cleared by a small fill
 * kernel ahead of the GEMM on `stream` (no memset node), so the call is legal under capture - once
 * the library knows where the array lives on that GPU: the first call with split_k > 1 on a device
 * looks the address up and must be made on a stream that is not capturing (under capture before
 * that it is refused with DFHIP_ERR_BAD_ARGUMENT and launches nothing).  The kernel is the one
 * dfhip_gemm_bf16_nt_splitk picks for the shape (its plan for a lone launch) with the caller's split_k. */
#define DFHIP_SPLITK_STATIC_BYTES ((64u << 20) + 4096u)
int dfhip_gemm_bf16_nt_splitk_static(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                     int64_t ldc, int M, int N, int K, int split_k,
                                     dfhip_stream_t stream);

/* C[M,N] = bf16( bf16(A W^T) + R ): the contraction with the residual addition
 * that follows it in a decoder layer (FX nodes linear, add of the host model traced by
 * examples/ae/scripts/bench_hf_transformers.py:206-210, run at dynaflow/runtime/engine.py:381) as the epilogue of the
 * kernel dfhip_gemm_bf16_plan picks.  R is [M,N] with the leading dimension of C;
 * the roundings are those of the separate linear and add kernels, so the bits are
 * the same.  split_k and workspace as in dfhip_gemm_bf16_nt_splitk (split_k = 1:
 * workspace may be null). */
int dfhip_gemm_bf16_nt_add(const void* A, int64_t lda, const void* W, int64_t ldw, const void* R, void* C,
                           int64_t ldc, int M, int N, int K, int split_k, void* workspace,
                           size_t workspace_bytes, dfhip_stream_t stream);

/* Gate and up projection with the SiLU*mul as the GEMM's epilogue:
 *   Out[M,I] = bf16( silu(A W_gate^T) * (A W_up^T) )
 * - the FX nodes linear, linear, silu, mul of the MLP (gate_proj and up_proj of
 * examples/ae/scheduler/hf/nanoflow.py:30, SiLU*mul as in examples/ae/up-silu-overlap.cu:75-90) in one
 * launch, the job of the reference's fused kernel (examples/ae/up-silu-overlap.cu:119-181).  Both
 * weights [I,K] with the same leading dimension ldw.  The epilogue applies
 * the roundings of the separate kernels (projections to bf16, silu to bf16,
 * product to bf16), so the result has the same bits as dfhip_gemm_bf16_nt
 * (K not split) twice + dfhip_silu_mul_bf16 with round_silu = 1.  Same shape
 * rules as dfhip_gemm_bf16_nt with N = I. */
int dfhip_gemm_bf16_gate_up_silu(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                 int64_t ldw, void* Out, int64_t ldo, int M, int I, int K,
                                 dfhip_stream_t stream);
/* The same for a launch that runs side by side with `share` - 1 others of its shape (see
 * dfhip_gemm_bf16_plan_shared; streams as assigned at examples/ae/scheduler/hf/nanoflow.py:122-146):
 * same result bits, the tile shape is chosen for the rounds the launches
 * take together. */
int dfhip_gemm_bf16_gate_up_silu_shared(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                        int64_t ldw, void* Out, int64_t ldo, int M, int I, int K,
                                        int share, dfhip_stream_t stream);

/* fp32 in / fp32 accumulate / fp32 out (the `linear` node, dynaflow/runtime/engine.py:381, of the
 * CPU-sized fp32 configuration).
 * Requires K % 4 == 0, 16-byte aligned pointers, lda/ldw % 4 == 0. */
int dfhip_gemm_f32_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                      int64_t ldc, int M, int N, int K, dfhip_stream_t stream);

/* fp8 e4m3fn inputs, fp32 accumulate, bf16 output (the `linear` node, dynaflow/runtime/engine.py:381,
 * of a host model whose weights are quantised per output channel and whose activations are
 * quantised per tensor):
 *   C[m,n] = bf16( a_scale[0] * w_scale[n] * sum_k A[m,k] * W[n,k] )
 * a_scale: device pointer to ONE float (per-tensor dynamic scale),
 * w_scale: device pointer to N floats (per-output-channel scale).
 * Requires K % 128 == 0, N % 8 == 0, lda/ldw % 16 == 0, ldc % 8 == 0. */
int dfhip_gemm_fp8_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                      int64_t ldc, const float* a_scale, const float* w_scale, int M, int N,
                      int K, dfhip_stream_t stream);
/* The same with an explicit kernel, for tuning and tests (the choice has no counterpart in the
 * reference): 0 = 256x256 LDS-DMA ring,
 * 1 = register-staged 128x128, 2 = 256x224 LDS-DMA ring (N = 7 * 2^k), negative =
 * the choice dfhip_gemm_fp8_nt makes. */
int dfhip_gemm_fp8_nt_variant(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                              const float* a_scale, const float* w_scale, int M, int N, int K, int variant,
                              dfhip_stream_t stream);
/* Gate and up projection of the fp8 MLP block with the SiLU*mul as the epilogue of ONE launch:
 *   g = bf16(a_scale * wg_scale[i] * A W_gate^T), u likewise with W_up,
 *   act[m,i] = bf16( silu(g) * u ),   amax[0] = max(amax[0], max |act|)
 * - the roundings of two dfhip_gemm_fp8_nt launches followed by dfhip_silu_mul_absmax_bf16, so the
 * same bits.  amax must hold 0 (or an earlier maximum) before the call; dfhip_quant_fp8_bf16 then
 * re-quantises act.  W_gate and W_up: [I, K] e4m3fn with one row stride.  In the reference these are
 * the FX nodes linear, linear, silu, mul of the host model's MLP (engine.py:381 runs them through
 * PyTorch); the wave-specialised fused kernel of examples/ae/OVERLAP.md:8-12 is the same idea. */
int dfhip_gemm_fp8_gate_up_silu_absmax(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                       int64_t ldw, void* act, int64_t ld_act, const float* a_scale,
                                       const float* w_gate_scale, const float* w_up_scale, float* amax, int M,
                                       int I, int K, dfhip_stream_t stream);

/* ------------------------------------------------------------ elementwise
 *
 * out[t,j] = bf16( (g / (1 + expf(-g))) * u ),  g = gate[t,j], u = up[t,j],
 * fp32 arithmetic, one rounding at the store - the `silu` and `mul` FX nodes,
 * written out in examples/ae/up-silu-overlap.cu:75-90.  `gate` and `up` have
 * their own row strides, so a packed gate_up[M, 2D] buffer is passed as
 * (gate = buf, up = buf + D, ld = 2D).  Requires D % 8 == 0, strides % 8 == 0.
 * With round_inputs_product != 0 the value silu(g) is first rounded to bf16
 * and then multiplied (what two separate bf16 aten kernels produce). */
int dfhip_silu_mul_bf16(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                        void* out, int64_t ld_out, int M, int D, int round_inputs_product,
                        dfhip_stream_t stream);

/* fp32 flavour of the same op (examples/ae/up-silu-overlap.cu:75-90 without the bf16 rounding; fp32
 * configuration). D % 4 == 0. */
int dfhip_silu_mul_f32(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                       void* out, int64_t ld_out, int M, int D, dfhip_stream_t stream);

/* RMSNorm over rows of x[M,H] (bf16), optional residual add:
 *   h = bf16(x + residual)            (residual may be NULL; written back to
 *                                      `residual_out` when that is not NULL)
 *   out = bf16( bf16(h * rsqrtf(mean(h^2) + eps)) * weight )
 * fp32 sum of squares; the arithmetic of
 * examples/ae/scheduler/vllm/tokenweave-kernels/csrc/tokenweave.cu:85-109
 * without its cross-GPU parts.  Requires H % 8 == 0 and H <= 16384. */
int dfhip_rmsnorm_bf16(const void* x, const void* residual, const void* weight, void* out,
                       void* residual_out, int M, int H, float eps, dfhip_stream_t stream);

/* Rotary position embedding of x[T, heads*head_dim] (bf16), Llama half-split
 * convention: pairs (x[i], x[i + head_dim/2]) of every head are rotated by the
 * angle of position (row % seq_len), cos/sin tables [seq_len, head_dim/2] fp32;
 * fp32 arithmetic, one rounding.  This is model code of the host framework in
 * the reference (it reaches DynaFlow as a chain of elementwise FX nodes that
 * dynaflow/runtime/engine.py:381 runs through PyTorch; examples/ae/MOE.md:29 counts it among the
 * "CUDA-bound" kernels of a step); here one launch.  head_dim % 16 == 0. */
int dfhip_rope_bf16(const void* x, int64_t ld_x, void* out, int64_t ld_out, const float* cos_table,
                    const float* sin_table, int T, int heads, int head_dim, int seq_len,
                    dfhip_stream_t stream);

/* Causal grouped-query attention for prefill (bf16, head_dim 128): B sequences of
 * S tokens each (S % 64 == 0), token t of sequence b is row b*S + t of q / k /
 * out; query head h sits at columns h*128 .. of a row, it reads kv head
 * h / (q_heads / kv_heads).  out = softmax(q k^T * scale, causal) v, scores in
 * fp32, probabilities rounded to bf16 for the second product, fp32 accumulation.
 * v is passed in the blocked layout v_blk[B][kv_heads][S/8][128][8] (8 consecutive
 * positions of one dim contiguous) that dfhip_pack_v_bf16 makes from v[B*S, ld_v].
 * One launch: a fast pass that never rescales its accumulators (a row's first
 * tile fixes the reference of its exponentials) and, in the workgroups where a
 * row's sum of exponentials ends beyond 2^64, a second pass with a running maximum.
 * In the reference this is the attention node of the host framework's model
 * graph (scaled_dot_product_attention of HF Llama, traced through
 * examples/ae/scripts/bench_hf_transformers.py:202-210); DynaFlow only schedules it. */
int dfhip_pack_v_bf16(const void* v, int64_t ld_v, void* v_blk, int B, int S, int kv_heads, int head_dim,
                      dfhip_stream_t stream);
int dfhip_causal_attention_bf16(const void* q, int64_t ld_q, const void* k, int64_t ld_k, const void* v_blk,
                                void* out, int64_t ld_o, int B, int S, int q_heads, int kv_heads, int head_dim,
                                float scale, dfhip_stream_t stream);

/* Decode step against a static KV cache (bf16, head_dim 128).  Cache layout, per
 * sequence slot and kv head, `capacity` positions (capacity % 32 == 0):
 *   k_cache [num_slots][kv_heads][capacity][128]
 *   v_cache [num_slots][kv_heads][capacity/8][128][8]   (8 consecutive positions
 *                                                       of one dim are contiguous)
 * Token t (one new token of sequence slot slots[t]) sits at position
 * lengths[t] - 1; lengths[t] is the number of positions it attends to, itself
 * included.  In the reference this is the host framework's attention custom op
 * with its paged cache (an FX node the schedulers treat as opaque:
 * examples/ae/scheduler/vllm/nanoflow.py:89-95 tags `unified_attention.*`
 * "attention", "no-cudagraph"); here
 * two kernels, or one that does both.
 *
 * dfhip_rope_kv_append_bf16: qkv[T, (q_heads + 2 kv_heads) * 128] holds q, k, v
 *   of the new tokens; q and k are rotated (half-split pairs, cos/sin tables
 *   [table_rows, 64] fp32, row = position), q goes to q_out[T, q_heads * 128], k
 *   and v are written into the caches.  Tokens with slot or position out of range
 *   leave the caches untouched.
 * dfhip_decode_attention_bf16: out[T, q_heads * 128] = softmax(q K^T * scale) V
 *   over positions 0 .. lengths[t]-1 of the token's slot, query head h reads kv
 *   head h / (q_heads / kv_heads); q_heads / kv_heads <= 16.  Every cached
 *   element is read once: HBM-bound.  A token whose slot is out of range or
 *   whose length is < 1 gets zeros.  Cache positions from lengths[t] on are never
 *   used, whatever they hold (uninitialised memory, NaN patterns).  A length
 *   beyond `capacity` is the caller's error and is not reported (nothing here
 *   synchronises): the append leaves the caches untouched and the token attends
 *   over the `capacity` cached positions, its own key and value not among them.
 * dfhip_decode_attention_append_bf16: both in ONE launch, same caches and same out bits as the two
 *   calls above: every (token, kv head) workgroup rotates its query heads in registers, rotates and
 *   appends its kv head's new key and value, and attends; the new key and value reach the products
 *   through LDS, not through a read of what was just written.  One launch less per layer and
 *   nano-batch of a decode step, and no q_out buffer.
 * The tokens of one call (and of calls that run at the same time) name distinct slots: a decode
 *   step has one new token per sequence, and two tokens of one slot would append to and read one
 *   cache concurrently. */
int dfhip_rope_kv_append_bf16(const void* qkv, int64_t ld_qkv, void* q_out, int64_t ld_q, void* k_cache,
                              void* v_cache, const int32_t* slots, const int32_t* lengths,
                              const float* cos_table, const float* sin_table, int T, int q_heads, int kv_heads,
                              int head_dim, int num_slots, int capacity, int table_rows, dfhip_stream_t stream);
int dfhip_decode_attention_bf16(const void* q, int64_t ld_q, const void* k_cache, const void* v_cache,
                                const int32_t* slots, const int32_t* lengths, void* out, int64_t ld_out, int T,
                                int q_heads, int kv_heads, int head_dim, int num_slots, int capacity, float scale,
                                dfhip_stream_t stream);
int dfhip_decode_attention_append_bf16(const void* qkv, int64_t ld_qkv, void* k_cache, void* v_cache,
                                       const int32_t* slots, const int32_t* lengths, const float* cos_table,
                                       const float* sin_table, void* out, int64_t ld_out, int T, int q_heads,
                                       int kv_heads, int head_dim, int num_slots, int capacity, int table_rows,
                                       float scale, dfhip_stream_t stream);

/* out[N,K] = in[K,N]^T for bf16 matrices: packs a weight kept as [in, out]
 * (x @ W convention) into the [out, in] layout the GEMMs read.  K, N % 8 == 0.  No counterpart in the
 * reference (torch.nn.functional.linear takes [out, in] weights as they are): a set-up helper. */
int dfhip_transpose_bf16(const void* in, int64_t ld_in, void* out, int64_t ld_out, int K, int N,
                         dfhip_stream_t stream);

/* ------------------------------------------------------------------- fp8
 *
 * Per-tensor dynamic quantisation of a bf16 activation to e4m3fn in two
 * launches: (1) amax[0] = max |x| (fp32; the caller zero-fills amax[0] before
 * the launch), (2) scale[0] = max(amax, 1e-12) / 448, q = e4m3fn(x / scale[0]),
 * round-to-nearest-even, saturating at +-448.  The reference ships no fp8 path of its own: these are
 * the quantisation nodes a host framework puts in front of an fp8 `linear` (run, like every node of a
 * sub-graph, at dynaflow/runtime/engine.py:381). */
int dfhip_absmax_bf16(const void* x, int64_t ld, int M, int D, float* amax,
                      dfhip_stream_t stream);
int dfhip_quant_fp8_bf16(const void* x, int64_t ld, void* q, int64_t ld_q, int M, int D,
                         const float* amax, float* scale_out, dfhip_stream_t stream);

/* silu(gate)*up in fp32 from bf16 inputs, written as bf16 to `out` (may be
 * NULL) and reduced into amax[0] = max |silu(g)*u| for the following
 * re-quantisation of the down-projection's input (the SiLU*mul of examples/ae/up-silu-overlap.cu:75-90
 * with the absmax that a per-tensor quantisation needs). */
int dfhip_silu_mul_absmax_bf16(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                               void* out, int64_t ld_out, int M, int D, float* amax,
                               dfhip_stream_t stream);

/* Fill `count` 32-bit words with `value` (a capture-safe replacement for
 * memset nodes, used to clear amax cells).  No counterpart in the reference (there a cudaMemset inside a
 * captured graph is fine, dynaflow/executor/cudagraph.py:84-122 captures whatever the callable issues). */
int dfhip_fill_u32(void* dst, uint32_t value, int64_t count, dfhip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DYNAFLOW_HIP_H */
