/*
 * coalsack_moe.h -- C ABI of the MI355X (gfx950) implementation of coalsack's
 * mixture-of-experts path: router -> dispatch -> MXFP4 expert MLP -> merge.
 *
 * Plain C, plain pointers and sizes.  Every function returns CSK_OK or an
 * error code; csk_last_error() gives the text for the calling thread.  No
 * exception crosses this boundary.  Citations name the reference interface
 * each entry point stands in for (paths relative to the reference root).
 *
 * Pointer conventions: "host" pointers are ordinary process memory, "device"
 * pointers come from csk_dev_alloc (or any hipMalloc).  All tensors are
 * row-major and contiguous, as dynamic_tensor is
 * (include/coalsack/tensor/dynamic_tensor.h:114-161).
 *
 * Threads: the library owns one GPU stream and one workspace, and serialises
 * its entry points with a process-wide lock; callers may come from any thread
 * (the reference drives each layer's nodes from that layer's scheduler thread,
 * include/coalsack/nn/model_io_nodes.h:224) and need no locking of their
 * own.  Device-pointer entry points are asynchronous on that stream; the
 * host-buffer ones return when their results are in place.
 */
#ifndef COALSACK_MOE_H
#define COALSACK_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CSK_OK 0
#define CSK_ERR_ARG 1          /* bad shape / null pointer / unsupported size   */
#define CSK_ERR_HIP 2          /* a HIP runtime call failed                      */
#define CSK_ERR_RANGE 3        /* expert index outside [0, E)                    */
#define CSK_ERR_ALL_EMPTY 4    /* merge: every expert tensor is empty            */
#define CSK_ERR_SCALE 5        /* MXFP4 scale byte 255 on a block with a code of magnitude >= 1 (overflows fp32) */
#define CSK_ERR_STATE 6        /* layer not fully populated                      */

/* expert_mlp_node::activation_type (include/coalsack/nn/nn_ops/expert_mlp_node.h:27-30) */
#define CSK_ACT_MODIFIED_SWIGLU 0
#define CSK_ACT_STANDARD_SWIGLU 1

/* which matrix of an expert */
#define CSK_W_UP 0
#define CSK_W_GATE 1
#define CSK_W_DOWN 2

/* csk_moe_forward flags */
#define CSK_FWD_RMSNORM 1  /* RMSNorm (csk_layer_set_norm) in front of router and experts */
#define CSK_FWD_RESIDUAL 2 /* out = hidden + moe(...)                                      */

typedef struct csk_layer csk_layer;   /* resident weights of one MoE layer */
typedef struct csk_mxfp4 csk_mxfp4;   /* one resident MXFP4 matrix         */

/* ---- process-wide ------------------------------------------------------ */

/* Select the GPU and create the library's stream.  Must precede everything
 * else; fails (CSK_ERR_HIP) when no gfx950 device is usable. */
int csk_init(int device);
const char* csk_last_error(void);
/* name (NUL-terminated, cap bytes), compute-unit count, total device memory */
int csk_device_info(char* name, size_t cap, int* compute_units, size_t* hbm_bytes);
/* free and total device memory as the runtime reports them now (either may be NULL) */
int csk_device_memory(size_t* free_bytes, size_t* total_bytes);
/* number of device allocations the library has made in this process so far (every one of
 * them goes through one counted call): unchanged across a call that allocates nothing */
int csk_alloc_count(uint64_t* count);

/* Device memory and timing for hosts with no HIP binding of their own. */
void* csk_dev_alloc(size_t bytes);
void csk_dev_free(void* p);
int csk_copy_h2d(void* dst_device, const void* src_host, size_t bytes);
int csk_copy_d2h(void* dst_host, const void* src_device, size_t bytes);
/* Device-to-device copy by a plain grid-stride kernel (16-byte accesses), asynchronous on the
 * library's stream; bytes must be a multiple of 16.  Also the known-size reference that profiler
 * byte counters are calibrated against. */
int csk_copy_d2d(void* dst_device, const void* src_device, size_t bytes);
int csk_synchronize(void);
typedef struct csk_event csk_event;
csk_event* csk_event_create(void);
void csk_event_destroy(csk_event* e);
int csk_event_record(csk_event* e);                 /* on the library's stream */
int csk_event_elapsed_ms(csk_event* a, csk_event* b, float* ms); /* waits for b */

/* Per-kernel timing of csk_moe_forward, for benchmarks: when enabled every
 * forward brackets its stages with events on the library's stream (a small
 * overhead, so throughput is measured with it off).  csk_stage_times waits for
 * the last forward and returns milliseconds per stage. */
#define CSK_STAGE_PREP 0     /* RMSNorm + activation split            */
#define CSK_STAGE_ROUTER 1   /* gate GEMV + top-k + softmax           */
#define CSK_STAGE_DISPATCH 2 /* histogram + scan + scatter            */
#define CSK_STAGE_GATEUP 3   /* gate/up projections + activation      */
#define CSK_STAGE_DOWN 4     /* down projection                       */
#define CSK_STAGE_COMBINE 5  /* weighted combine (+ residual)         */
#define CSK_N_STAGES 6
int csk_stage_timing(int enable);
int csk_stage_times(float* ms_out);
/* With stage timing enabled, the gate/up and the down kernel of an MXFP4 layer carry a
 * start and a stop event on the dispatch itself: ms_out[0], ms_out[1] are their own
 * begin-to-end durations in the last forward -- the figure a kernel trace reports, without
 * the cost of the events recorded between launches that csk_stage_times includes. */
int csk_kernel_times(float* ms_out2);

/* ---- resident MXFP4 matrices ------------------------------------------- */

/* Take a [rows, K] matrix in the reference's storage format -- rows of K/32
 * consecutive 17-byte blocks, scale byte first, byte j carrying element j in
 * the low nibble and element j+16 in the high nibble
 * (include/coalsack/tensor/dynamic_mx_tensor.h:19-45,
 *  include/coalsack/gguf/gguf_dequant.h:437-455) -- and keep a repacked copy in
 * HBM.  Replaces what moe_weight_provider::get returns for one expert tensor
 * (src/llm/moe_weight_provider.cpp:160-188).  K % 32 == 0. */
int csk_mxfp4_upload(const uint8_t* blocks17_host, int64_t rows, int64_t K, csk_mxfp4** out);
void csk_mxfp4_free(csk_mxfp4* m);
/* Dequantise the resident copy on the GPU into host_out[rows*K]; bit-identical
 * to dequantize_block_mxfp4 (gguf_dequant.h:437-455) for every scale byte the upload
 * accepts: 0..254, and 255 on blocks whose codes are all 0 or +-0.5 (the finite values of
 * that byte, 0 and +-2^127; kept as byte 254 with the codes doubled, which is how
 * csk_mxfp4_export and csk_layer_export return such a block; any larger code under byte 255
 * is an infinity in the reference and is refused with CSK_ERR_SCALE).  Blocks with scale bytes 0 and 1
 * hold fp32 denormals (|w| <= 12 * 2^-127); the expert kernels contract them as zeros. */
int csk_mxfp4_dequant(const csk_mxfp4* m, float* host_out);
/* Recover the 17-byte blocks from the resident copy (round-trip check). */
int csk_mxfp4_export(const csk_mxfp4* m, uint8_t* blocks17_host);

/* ---- resident fp16 matrices ---------------------------------------------- */

/* A [rows, K] row-major matrix of IEEE halves, as expert_mlp_node::compute_fp16
 * receives w_up / w_gate / w_down (expert_mlp_node.h:269-389: dtype::float16,
 * 2-D) and as moe_weight_provider::get produces them from F16, Q4_K or Q6_K
 * checkpoints (src/llm/moe_weight_provider.cpp:134-159).  Kept in HBM as
 * 16 x 32 tiles in matrix-instruction order; no value changes.  Any rows, K
 * in 1..65536. */
typedef struct csk_f16 csk_f16;
int csk_f16_upload(const uint16_t* halves_host, int64_t rows, int64_t K, csk_f16** out);
void csk_f16_free(csk_f16* m);
/* The same from a matrix stored as ggml type F16 (1), Q4_K (12) or Q6_K (14): K-quant
 * streams are widened to fp16 exactly as moe_weight_provider::get does
 * (src/llm/moe_weight_provider.cpp:17-33, 134-159: dequantize_block_q4_K / q6_K, then
 * fp32_to_fp16 -- the truncating conversion of a build without F16C,
 * include/coalsack/gguf/gguf_dequant.h:149-258, 458-487).  rows * K must be a multiple
 * of 256 for the K-quants. */
int csk_f16_upload_ggml(int ggml_type, const void* data_host, int64_t rows, int64_t K, csk_f16** out);
/* The same from a row-major fp32 matrix -- the FLOAT32 weights dense_ffn_node and
 * matmul_transpose_mixed_node also accept (dense_ffn_node.h:57-60, 101-114;
 * matmul_transpose_mixed_node.h:29-31, 91-101).  Kept as two fp16 terms side by side,
 * [rows, 2 K] = [fp16(w') | fp16(w' - fp16(w'))] with w' = w / 2^s, one power of two per
 * matrix that brings its largest magnitude into [2^14, 2^15) and that the kernels multiply
 * back into their sums: 22 significant bits for every weight down to 2^-18 of the largest,
 * whatever the magnitude of the matrix.  Contracted against each activation row twice
 * over, so the fp16 kernels serve both kinds.  Any finite fp32 is accepted; a NaN or an
 * infinity is refused.  Accepted by csk_dense_ffn_f16 and csk_matmul_transpose_f16. */
int csk_f16_upload_f32(const float* w_host, int64_t rows, int64_t K, csk_f16** out);
/* Recover the row-major halves from the resident copy (round-trip check); [rows, 2 K] (the
 * two terms of w / 2^s) for a matrix that came in as fp32. */
int csk_f16_export(const csk_f16* m, uint16_t* halves_host);

/* ---- one MoE layer, weights resident ------------------------------------ */

/* E experts, top-k, hidden size H, expert intermediate size F.  H and F must
 * be multiples of 32 (expert_mlp_node.h:463-472). */
int csk_layer_create(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out);
void csk_layer_destroy(csk_layer* L);
/* moe_router_node::set_sigmoid_gating (moe_router_node.h:34),
 * expert_mlp_node::set_activation_type / set_weight_before_ffn
 * (expert_mlp_node.h:47-52), expert_merge_node::set_weight_before_ffn
 * (expert_merge_node.h:24). */
int csk_layer_set_options(csk_layer* L, int sigmoid_gating, int activation, int weight_before_ffn);
/* gate_w [E,H] f32, gate_b [E] f32 or NULL (moe_router_node.h:51-124 inputs 1,2) */
int csk_layer_set_router(csk_layer* L, const float* gate_w_host, const float* gate_b_host);
/* One expert's tensors as moe_weight_fetch_node hands them to expert e
 * (moe_weight_fetch_node.h:189-206): w_up/w_gate [F,H], w_down [H,F] in
 * 17-byte blocks; biases f32 [F],[F],[H] or all NULL. */
int csk_layer_set_expert(csk_layer* L, int64_t e, const uint8_t* w_up, const uint8_t* w_gate,
                         const uint8_t* w_down, const float* b_up, const float* b_gate,
                         const float* b_down);
/* rmsnorm_node weight [H] and epsilon (rmsnorm_node.h:62-83) */
int csk_layer_set_norm(csk_layer* L, const float* weight_host, float eps);
/* Fill every expert's three matrices on the GPU from a counter-based
 * generator (no host copy): block b of stream (seed, layer_index, expert,
 * matrix) gets scale byte scale_lo + h0 % scale_span and 16 quant bytes from
 * h1, h2, with h_i = splitmix64 finaliser of (stream_key + 3 b + i).  A host
 * can replay any slice.  Biases are left as set (or absent). */
int csk_layer_fill_synthetic(csk_layer* L, uint64_t seed, int64_t layer_index, int scale_lo,
                             int scale_span);
int csk_layer_dequant(const csk_layer* L, int64_t e, int which, float* host_out);
int csk_layer_export(const csk_layer* L, int64_t e, int which, uint8_t* blocks17_host);

/* The same layer with fp16 experts: the other branch of expert_mlp_node::process
 * (expert_mlp_node.h:269-389, compute_token :533-647), which the engine takes for
 * checkpoints whose expert tensors are F16, Q4_K or Q6_K
 * (src/llm/moe_weight_provider.cpp:134-159).  Router, options, norm, forward and
 * csk_layer_fill_synthetic (halves j / 2^14, j uniform in [-2048, 2047]) work as
 * for an MXFP4 layer; the weights come in through csk_layer_set_expert_f16:
 * row-major halves w_up/w_gate [F,H], w_down [H,F]; biases f32 or all NULL. */
int csk_layer_create_f16(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out);
int csk_layer_set_expert_f16(csk_layer* L, int64_t e, const uint16_t* w_up, const uint16_t* w_gate,
                             const uint16_t* w_down, const float* b_up, const float* b_gate,
                             const float* b_down);
/* One matrix of expert e (which = CSK_W_UP / CSK_W_GATE / CSK_W_DOWN) from ggml type
 * F16, Q4_K or Q6_K data, as csk_f16_upload_ggml; a checkpoint may mix the three. */
int csk_layer_set_expert_matrix(csk_layer* L, int64_t e, int which, int ggml_type, const void* data_host);
int csk_layer_export_f16(const csk_layer* L, int64_t e, int which, uint16_t* halves_host);

/* ---------------------------------------------------------------- GGUF ingest
 * Reads a GGUF file's key/value section and tensor table (no tensor data) --
 * gguf_loader::load, src/gguf/gguf_loader.cpp:383-518.  Needs no GPU and no
 * csk_init. */
typedef struct csk_gguf csk_gguf;
int csk_gguf_open(const char* path, csk_gguf** out);
/* A split checkpoint: the shards in order, merged as gguf_multi_loader::load does
 * (src/gguf/gguf_multi_loader.cpp:25-76, used by src/llm/moe_weight_provider.cpp:75-100):
 * a tensor belongs to the shard that lists it (a name in two shards is an error), a metadata
 * key is answered by the first shard that has it.  csk_layer_from_gguf then reads every
 * tensor from its own shard. */
int csk_gguf_open_shards(const char* const* paths, int64_t n_paths, csk_gguf** out);
void csk_gguf_close(csk_gguf* g);
int csk_gguf_tensor_count(const csk_gguf* g, int64_t* n);
int csk_gguf_tensor_name(const csk_gguf* g, int64_t index, char* buf, size_t cap);
/* gguf_loader::get_tensor_info: dims in file order (fastest-varying first, padded
 * with 1), absolute file offset of the data, size in bytes (0: unknown type). */
int csk_gguf_tensor_info(const csk_gguf* g, const char* name, uint32_t* ggml_type, int32_t* n_dims,
                         uint64_t* dims4, uint64_t* file_offset, uint64_t* nbytes);
/* gguf_multi_loader::tensor_info::shard_idx: which file of a split checkpoint holds the tensor (0 for a single file) */
int csk_gguf_tensor_shard(const csk_gguf* g, const char* name, int32_t* shard);
/* gguf_loader::get_uint32 / get_string (any integer width is accepted) */
int csk_gguf_get_u32(const csk_gguf* g, const char* key, uint32_t* value);
int csk_gguf_get_str(const csk_gguf* g, const char* key, char* buf, size_t cap);
/* Resident MoE layer of transformer block `block`, built from
 *   blk.N.ffn_gate_inp.{weight,bias}, blk.N.ffn_{up,gate,down}_exps.{weight,bias},
 *   blk.N.post_attention_norm.weight (llama4: ffn_norm.weight)
 * with <arch>.expert_count / expert_used_count and the architecture switches of
 * llm_engine::load_config_from_gguf (src/llm/llm_engine.cpp:135-225).  Expert e
 * of a stacked tensor is the slice at offset + e * rows * (K/32) * 17 --
 * moe_weight_provider::get, src/llm/moe_weight_provider.cpp:160-188; it takes
 * the place of that provider and its LRU cache: all experts stay in HBM.
 * Expert tensors are MXFP4, or F16 / Q4_K / Q6_K (a layer with fp16 experts,
 * as moe_weight_provider.cpp:134-159 hands them to the node). */
int csk_layer_from_gguf(csk_gguf* g, int64_t block, csk_layer** out);

/* Router -> dispatch -> expert MLPs -> merge for T tokens, everything on the
 * GPU: hidden and out are device pointers [T,H] f32 (out may be hidden itself:
 * the layer then updates the rows in place).  Stands in for the node chain
 * llm_engine wires per layer (src/llm/llm_engine.cpp:714-777).  Asynchronous on
 * the library's stream.  Any T: a batch longer than the pass size (32768 tokens
 * unless csk_set_pass_tokens changed it) is taken in several passes of equal
 * size -- tokens do not depend on one another -- so the workspace stays bounded. */
int csk_moe_forward(csk_layer* L, const float* hidden_device, int64_t T, float* out_device,
                    int flags);
/* csk_moe_forward for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments, same kernels and the same results bit for bit, but every
 * intermediate buffer lives in a device array that is part of the library image (21 MB per
 * GPU, held until the process ends), and the call makes no hipMalloc / hipFree.  Limits:
 * MXFP4 layers, T <= 64 tokens, T * top_k <= 512, hidden_dim and expert_ffn_dim <= 3072;
 * anything larger is refused with CSK_ERR_ARG.  All calls on a GPU share that array (it keeps
 * the previous call's contents; nothing in it has to start at zero): calls that overlap on
 * one GPU would race -- the library's lock and single stream order them. */
int csk_moe_forward_noalloc(csk_layer* L, const float* hidden_device, int64_t T, float* out_device,
                            int flags);
/* Largest number of tokens one pass of csk_moe_forward takes (1..65536). */
int csk_set_pass_tokens(int64_t tokens);
/* Same through host buffers; also returns the router output [T,k,2] when
 * pairs_out is not NULL.  Synchronous. */
int csk_moe_forward_host(csk_layer* L, const float* hidden, int64_t T, float* out, float* pairs_out,
                         int flags);
/* n layers in sequence, each h <- h + moe(rmsnorm(h)); hidden_device [T,H] is
 * updated in place. */
int csk_moe_stack_forward(csk_layer* const* layers, int64_t n_layers, float* hidden_device,
                          int64_t T);
/* ---- one MoE block behind the reference's node classes (src/llm/llm_engine.cpp:721-753,
 * include/coalsack/llm/graph_builder.h:289-372: router node -> weight fetch -> one expert
 * node per expert -> merge node).  The expert nodes own the resident matrices; a view layer
 * points at them, and a frame runs the block as csk_moe_forward_host does while every node
 * still emits what the reference's node emits. */
/* A layer without expert matrices of its own (router, biases and norm as any layer). */
int csk_layer_create_view(int64_t E, int64_t k, int64_t H, int64_t F, csk_layer** out);
/* Expert e of a view := these three resident matrices (owned by the caller: detach before
 * freeing one) and these biases (host pointers, copied; all three or none). */
int csk_layer_attach_expert(csk_layer* L, int64_t e, const csk_mxfp4* up, const csk_mxfp4* gate,
                            const csk_mxfp4* down, const float* b_up, const float* b_gate,
                            const float* b_down);
int csk_layer_detach_expert(csk_layer* L, int64_t e);
/* moe_router_node's part (moe_router_node.h:51-124): uploads hidden [T,H] (host), runs router
 * and dispatch, returns the router output [T,k,2] in pairs_out; if every expert the frame
 * selects is attached, the experts and the merge are then started on the device and
 * *experts_running is 1 (else 0: the expert nodes compute on their own, as without a view). */
int csk_moe_frame_begin(csk_layer* L, const float* hidden, int64_t T, float* pairs_out, int flags,
                        int* experts_running);
/* expert_mlp_node's part (expert_mlp_node.h:503-529): into out [T,H] (host, zero-filled by the
 * caller) the rows of the tokens that selected expert e -- what the node emits.  The first
 * call of a frame waits for the experts and fetches all rows at once. */
int csk_moe_frame_expert_rows(csk_layer* L, int64_t e, float* out);
/* An expert node found that its weights are no longer the attached ones and computed its
 * output itself: the frame's merged rows must not be used. */
int csk_moe_frame_void(csk_layer* L);
/* expert_merge_node's part (expert_merge_node.h:30-134): the merged rows [T,H] of the frame
 * if its experts ran and nothing voided it (*available = 1), bit-identical to
 * csk_moe_forward_host; else *available = 0 and out is untouched. */
int csk_moe_frame_merged(csk_layer* L, float* out, int* available);

/* Intermediate results of the last csk_moe_forward on L, for tests:
 * per-expert token counts [E] and the packed token list (token ids grouped by
 * expert, ascending within an expert) [T*k]. */
int csk_layer_last_dispatch(csk_layer* L, int32_t* counts_host, int32_t* tokens_host);

/* ---- node-level operations through host buffers -------------------------- */

/* moe_router_node::compute (moe_router_node.h:51-214): hidden [T,H], gate_w
 * [E,H], gate_b [E] or NULL -> out_pairs [T,k,2] = (expert index as float,
 * weight). */
int csk_moe_router(const float* hidden, int64_t T, int64_t H, const float* gate_w, int64_t E,
                   const float* gate_b, int64_t k, int sigmoid_gating, float* out_pairs);
/* The same router for a caller that keeps the gate in device memory between frames
 * (moe_router_node is handed the same gate tensors every frame): gate_w_dev [E,H] and
 * gate_b_dev [E] or NULL are device pointers (csk_dev_alloc + csk_copy_h2d); hidden and
 * out_pairs stay host pointers.  Replaces the same lines of the reference as
 * csk_moe_router. */
int csk_moe_router_resident(const float* hidden, int64_t T, int64_t H, const float* gate_w_dev,
                            int64_t E, const float* gate_b_dev_or_null, int64_t k,
                            int sigmoid_gating, float* out_pairs);
/* The logits of that router as this library first computes them (fp32, tree-ordered
 * sums; [T,E]), before any recomputation in the reference's summation order -- a
 * diagnostic: the tests bound their distance from the reference's sequential sums,
 * which is what the close-call threshold of the top-k selection rests on. */
int csk_moe_router_logits(const float* hidden, int64_t T, int64_t H, const float* gate_w, int64_t E,
                          const float* gate_b_or_null, float* out_logits);
/* expert_mlp_node::compute_with_mxfp4 for one expert (expert_mlp_node.h:392-530):
 * out [T,H]; *is_empty = 1 and out untouched when no token selected expert_id
 * (:441-443); rows of unselected tokens are zero (:509-512). */
int csk_expert_mlp_mxfp4(int expert_id, const float* hidden, int64_t T, int64_t H, int64_t F,
                         const csk_mxfp4* w_up, const csk_mxfp4* w_gate, const csk_mxfp4* w_down,
                         const float* b_up, const float* b_gate, const float* b_down,
                         const float* router_pairs, int64_t k, int activation,
                         int weight_before_ffn, float* out, int* is_empty);
/* expert_mlp_node::compute_fp16 for one expert (expert_mlp_node.h:269-389,
 * token loop :740-780): conventions of csk_expert_mlp_mxfp4; H and F need not be
 * multiples of anything (the reference's rows end in a scalar remainder loop,
 * :578-585). */
int csk_expert_mlp_f16(int expert_id, const float* hidden, int64_t T, int64_t H, int64_t F,
                       const csk_f16* w_up, const csk_f16* w_gate, const csk_f16* w_down,
                       const float* b_up, const float* b_gate, const float* b_down,
                       const float* router_pairs, int64_t k, int activation,
                       int weight_before_ffn, float* out, int* is_empty);
/* dense_ffn_node::compute with float16 weights (include/coalsack/nn/nn_ops/dense_ffn_node.h:
 * 36-118, compute_token :163-218): the shared expert of llama4-style blocks
 * (src/llm/llm_engine.cpp:755-771) -- every token through one gated MLP with the standard
 * SwiGLU.  out [T,H]; w_gate/w_up [F,H], w_down [H,F]; each bias f32 or NULL.  Any H, F. */
int csk_dense_ffn_f16(const float* hidden, int64_t T, int64_t H, int64_t F, const csk_f16* w_gate,
                      const csk_f16* w_up, const csk_f16* w_down, const float* b_gate,
                      const float* b_up, const float* b_down, float* out);
/* matmul_transpose_mixed_node::compute with a 2-D float16 weight
 * (include/coalsack/nn/nn_ops/matmul_transpose_mixed_node.h:25-110, compute_matmul_avx2_fp16b
 * :198-308): out [M,N] = A [M,K] (fp32, leading dimensions flattened) x W [N,K]^T -- the
 * engine's linear projections (include/coalsack/llm/graph_builder.h:90-105). */
int csk_matmul_transpose_f16(const float* a_host, int64_t M, int64_t K, const csk_f16* w, float* out_host);
/* expert_mlp_node::compute_test_mxfp4 (expert_mlp_node.h:63-70): one token,
 * raw 17-byte-block weights in host memory. */
int csk_expert_token_mxfp4(const float* hidden_vec, const uint8_t* w_up, const uint8_t* w_gate,
                           const uint8_t* w_down, const float* b_up, const float* b_gate,
                           const float* b_down, float* out_vec, int64_t H, int64_t F,
                           int activation);
/* expert_merge_node::compute (expert_merge_node.h:30-134): expert_outs[e] is a
 * host [T,H] tensor or NULL for an empty one. */
int csk_expert_merge(const float* router_pairs, int64_t T, int64_t k, int64_t E, int64_t H,
                     const float* const* expert_outs, int pre_weighted, float* out);
/* rmsnorm_node::compute (rmsnorm_node.h:62-83) and add_node (add_node.h:8-55) */
int csk_rmsnorm(const float* x, const float* weight, float* out, int64_t T, int64_t H, float eps);
/* the node's float64 branch (rmsnorm_node.h:49-50, compute_impl<double>): input, weight and
 * output are doubles; sums, division, square root and products in double, in the
 * reference's order -- the result equals the CPU's bit for bit */
int csk_rmsnorm_f64(const double* x, const double* weight, double* out, int64_t T, int64_t H, float eps);
int csk_add(const float* a, const float* b, float* out, int64_t n);
/* add_node over operands of different shapes and of the node's other element types
 * (add_node.h:16-50 through elementwise_binary_op, elementwise_helpers.h:9-66): numpy-style
 * broadcasting over trailing dimensions as dynamic_tensor::broadcast_shape defines it
 * (dynamic_tensor.h:218-238).  dtype is one of CSK_DT_*; both operands and the result have
 * it.  `out` holds the broadcast shape's element count.  Shapes that do not broadcast return
 * CSK_ERR_ARG with the reference's text "Broadcast failed: Shape A=[..], Shape B=[..]".  At
 * most 8 dimensions.  Integer sums wrap. */
#define CSK_DT_FLOAT32 0
#define CSK_DT_FLOAT64 1
#define CSK_DT_INT32 2
#define CSK_DT_INT64 3
int csk_add_broadcast(const void* a, const int64_t* shape_a, int nd_a, const void* b,
                      const int64_t* shape_b, int nd_b, int dtype, void* out);
/* moe_router_node::compute_impl<double> (moe_router_node.h:115-118, 141-214): float64 hidden
 * states [T,H] and gate weights [E,H], float32 bias [E] or NULL; logits are the reference's
 * sequential float64 sums bit for bit, selection runs on them, weights and the [T,k,2]
 * output are float32.  out_logits ([T,E] float64) may be NULL. */
int csk_moe_router_f64(const double* hidden, int64_t T, int64_t H, const double* gate_w, int64_t E,
                       const float* gate_b, int64_t k, int sigmoid, float* out_pairs,
                       double* out_logits);

#ifdef __cplusplus
}
#endif
#endif /* COALSACK_MOE_H */
