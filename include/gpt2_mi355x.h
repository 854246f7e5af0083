/*
 * C ABI of the MI355X (gfx950) GPT-2 fp32 forward library, libgpt2_mi355x.so.
 *
 * The entry points keep the llm.c launcher convention that the reference's
 * kernels are drop-ins for: raw device pointers + int dims, caller owns every
 * buffer, launches go to the null stream in order, nothing synchronises and
 * nothing is allocated inside a launcher.  Each launcher exists in two forms:
 *
 *   int  <name>_status(...)   returns 0 or a GPT2HIP_E* code (message via
 *                             gpt2hip_last_error()); never aborts.
 *   void <name>(...)          the llm.c form: prints the message and aborts on
 *                             failure, like llm.c's cudaCheck / the reference's
 *                             assert()s.
 *
 * All tensors are fp32, row-major, device memory.  Rows do not need padding.
 */
#ifndef GPT2_MI355X_H
#define GPT2_MI355X_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  GPT2HIP_OK = 0,
  GPT2HIP_EINVAL = 1, /* bad shape or null pointer */
  GPT2HIP_EHIP = 2,   /* a HIP runtime call failed */
  GPT2HIP_ENOMEM = 3
};

/* Message of the last failure on the calling thread ("" if none). */
const char* gpt2hip_last_error(void);

/* out[b,t,:] = wte[inp[b,t],:] + wpe[t,:].  inp is int32 (B,T) on the device.
 * Replaces llm.c's encoder_forward, which the reference leaves untouched
 * (named in reference README.md:10). */
int encoder_forward_status(float* out, const int* inp, const float* wte, const float* wpe, int B,
                           int T, int C);
void encoder_forward(float* out, const int* inp, const float* wte, const float* wpe, int B, int T,
                     int C);

/* Row-wise layernorm, eps 1e-5; mean/rstd (B*T) may be NULL.
 * Replaces layernorm_forward_warp, reference
 * kernels/layernorm/3_layernorm_warp.cuh:78-80. */
int layernorm_forward_status(float* out, float* mean, float* rstd, const float* inp,
                             const float* weight, const float* bias, int B, int T, int C);
void layernorm_forward(float* out, float* mean, float* rstd, const float* inp, const float* weight,
                       const float* bias, int B, int T, int C);

/* res_out = inp1 + inp2; layernorm_out = layernorm(res_out); mean/rstd may be
 * NULL.  res_out may alias inp1 or inp2.  Replaces
 * fused_residual_layernorm_forward, reference
 * kernels/fused_residual_layernorm/fused_residual_layernorm.cuh:88-90. */
int fused_residual_layernorm_forward_status(float* res_out, float* layernorm_out, float* mean,
                                            float* rstd, const float* inp1, const float* inp2,
                                            const float* weight, const float* bias, int B, int T,
                                            int C);
void fused_residual_layernorm_forward(float* res_out, float* layernorm_out, float* mean,
                                      float* rstd, const float* inp1, const float* inp2,
                                      const float* weight, const float* bias, int B, int T, int C);

/* out = inp1 + inp2 over N floats.  Replaces residual_forward_naive, reference
 * kernels/residual/1_residual_naive.cuh:15. */
int residual_forward_status(float* out, const float* inp1, const float* inp2, int N);
void residual_forward(float* out, const float* inp1, const float* inp2, int N);

/* tanh-GELU over N floats (llm.c's gelu_forward; the reference only has the
 * device function, kernels/matmul/9_matmul_async_cg_tf32_gelu.cuh:5-11).
 * size_t form for N above INT_MAX is not needed at GPT-2 sizes. */
int gelu_forward_status(float* out, const float* inp, int N);
void gelu_forward(float* out, const float* inp, int N);

/* out(B*T,OC) = inp(B*T,C) . weight(OC,C)^T + bias(OC); bias may be NULL.
 * Any B*T, C, OC >= 1.  Replaces matmul_forward_cublas, reference
 * kernels/matmul/2_matmul_cublas.cuh:34-42 (and the other numbered attempts,
 * which share the signature). */
int matmul_forward_status(float* out, const float* inp, const float* weight, const float* bias,
                          int B, int T, int C, int OC);
void matmul_forward(float* out, const float* inp, const float* weight, const float* bias, int B,
                    int T, int C, int OC);

/* Which workgroup tile (rows x columns of the product) matmul_forward gives a problem:
 * 256x192, 256x128, 128x192, 128x160 (only where OC is a multiple of 160), 128x128, 128x96,
 * 64x128, 64x96, 64x64 or 32x32, chosen by a fitted
 * cost model so that the tiles come out in close to whole rounds over the 256 compute units
 * (the reference launches one fixed 128x128 tile shape and asserts divisibility,
 * kernels/matmul/9_matmul_async_cg_tf32_gelu.cuh:266-274).  Both are 0 for problems that
 * take another kernel (C % 32 != 0, B*T <= 16).  A product of 1536 or more columns whose tiles
 * come out just above a whole number of rounds (the lm-head at up to a few thousand rows, a
 * 2304-wide product at 1024 rows) is computed by two launches over ranges of its columns --
 * whole rounds of one tile, then the columns left, at most a quarter, with whatever suits
 * those; the shape reported is the first launch's.
 * Touches no GPU. */
int matmul_forward_tile_shape(int B, int T, int C, int OC, int* tile_rows, int* tile_cols);

/* How many of the OC columns the first of those two launches computes (OC: the product is one
 * launch; 0: bad arguments).  workspace_bytes as for matmul_forward_splitk_plan.  Touches no GPU. */
int matmul_forward_first_columns(int B, int T, int C, int OC, size_t workspace_bytes);

/* Same with tanh-GELU applied to the result when is_gelu != 0.  Replaces
 * matmul_forward_async_cg_tf32_gelu, reference
 * kernels/matmul/9_matmul_async_cg_tf32_gelu.cuh:237-246. */
int matmul_forward_gelu_status(float* out, const float* inp, const float* weight,
                               const float* bias, int B, int T, int C, int OC, int is_gelu);
void matmul_forward_gelu(float* out, const float* inp, const float* weight, const float* bias,
                         int B, int T, int C, int OC, int is_gelu);

/* matmul_forward_gelu for a caller that can lend a workspace: with it the K dimension of a
 * tile can be split between several workgroups, whose partial tiles meet in the workspace and
 * are summed in a fixed order by whichever workgroup of the tile finishes last (results do not
 * depend on timing; they differ from matmul_forward's by fp32 rounding of the summation
 * order).  This is what fills the 256 compute units when a problem has too few tiles, or a
 * tile count just above a multiple of 256 -- the "wave quantisation" that the reference's
 * fixed grid of one 128x128 tile per block leaves in place
 * (kernels/matmul/9_matmul_async_cg_tf32_gelu.cuh:266-274).  Whether and how K is split is
 * chosen by the same fitted cost model as the tile shape; without a workspace (NULL / 0) the
 * call is matmul_forward_gelu.
 * workspace: device memory, 256-byte aligned.  Its first GPT2HIP_SPLITK_COUNTER_BYTES are
 * per-tile counters: zero them once (hipMemset) before the first call; every call leaves them
 * zero.  The rest holds partial tiles (tiles x splits x tile area x 4 bytes; a plan that does
 * not fit is not chosen).  matmul_forward_splitk_workspace() is a size that never constrains
 * the choice at GPT-2 shapes.  Calls that overlap on one GPU need a workspace each.  If a
 * launch that used the workspace did not run to completion (a device error), zero the
 * counters again before reusing it. */
#define GPT2HIP_SPLITK_COUNTER_BYTES 16384u
size_t matmul_forward_splitk_workspace(void);
int matmul_forward_splitk_status(float* out, const float* inp, const float* weight, const float* bias,
                                 int B, int T, int C, int OC, int is_gelu, void* workspace,
                                 size_t workspace_bytes);
/* out = resid + (inp . weight^T + bias): the product with a transformer block's residual add in
 * its epilogue (every workgroup reads the entries of resid that match the tile it is about to
 * store), so that the add costs no pass of its own over memory.  The reference adds the
 * residual in the kernel that also normalises (kernels/layernorm/fused_residual_layernorm.cuh:
 * 88-90, which fused_residual_layernorm_forward keeps as a launcher); the library's gpt2_forward
 * driver adds it here instead and runs layernorm_forward on the sum: the same additions in the
 * same order, bit for bit, with half the normalisation kernel's traffic.  resid: (B*T, OC), must
 * not overlap out.  workspace as for matmul_forward_splitk_status (NULL / 0: none). */
int matmul_forward_residual_status(float* out, const float* inp, const float* weight, const float* bias,
                                   const float* resid, int B, int T, int C, int OC, void* workspace,
                                   size_t workspace_bytes);
/* The plan matmul_forward_splitk_status would choose: tile shape (0 x 0 for problems outside
 * the tiled kernels) and workgroups per tile (1 = K not split).  Touches no GPU. */
int matmul_forward_splitk_plan(int B, int T, int C, int OC, size_t workspace_bytes, int* tile_rows,
                               int* tile_cols, int* splits);
/* The same product with the plan given by the caller (tile shape one of those listed at
 * matmul_forward_tile_shape, 1 <= splits <= C / 32): for parity tests of every kernel form
 * and for the sweeps that the cost model is fitted to.  Needs C % 32 == 0. */
int matmul_forward_splitk_forced_status(float* out, const float* inp, const float* weight,
                                        const float* bias, int B, int T, int C, int OC, int is_gelu,
                                        void* workspace, size_t workspace_bytes, int tile_rows,
                                        int tile_cols, int splits);

/* Diagnostic form of matmul_forward (C % 32 == 0, 16-byte aligned operands): the
 * same kernel, which also stores for each of its workgroups four 64-bit words in
 * probe[] (device memory, probe_capacity workgroups): wall clock (100 MHz) at the
 * start and end of the K loop, then the shader clock at the same two instants.
 * *workgroups receives the number of workgroups launched (at most
 * ceil(B*T/32) * ceil(OC/32), which probe_capacity must cover).  No counterpart in the
 * reference; it separates instruction-issue efficiency from the clock frequency the
 * chip sustains under the load. */
int matmul_forward_probe_status(float* out, const float* inp, const float* weight,
                                const float* bias, int B, int T, int C, int OC,
                                unsigned long long* probe, int probe_capacity, int* workgroups);

/* Causal multi-head self-attention.  inp is packed qkv (B,T,3C): q at column
 * 0, k at +C, v at +2C, head h at h*(C/NH) inside each; out is (B,T,C).
 * qkvr and att are the llm.c scratch arguments: ignored, may be NULL.  inp is
 * never written.  Replaces flash_attention_permute_forward, reference
 * kernels/attention/3_flash_attention_permute.cuh:346-351. */
int attention_forward_status(float* out, float* qkvr, float* att, const float* inp, int B, int T,
                             int C, int NH);
void attention_forward(float* out, float* qkvr, float* att, const float* inp, int B, int T, int C,
                       int NH);

/* ids[r] = argmax_v logits[r,v] for N rows of V floats; lowest index wins ties.
 * No counterpart in the reference (llm.c samples on the host); needed for the
 * "argmax ids" output of the forward pass. */
int argmax_forward_status(int* ids, const float* logits, int N, int V);
void argmax_forward(int* ids, const float* logits, int N, int V);

/* matmul_forward followed by argmax_forward without the (B*T, OC) product ever reaching
 * memory: ids[r] = argmax_o (inp[r,:] . weight[o,:] + bias[o]), lowest index wins ties.
 * For C % 32 == 0 and 16-byte aligned operands (the lm-head) the GEMM's tiles are reduced
 * to (value, column) pairs in their epilogue and a second small kernel reduces the pairs.
 * The products are accumulated over C in ascending order, as every tiled kernel of
 * matmul_forward accumulates them, so wherever matmul_forward does not split C between
 * waves the ids equal argmax_forward over matmul_forward's output bit for bit (it splits C
 * for B*T <= 16, for 32x32 tiles and for up to 512 tiles of 64x64: small problems; a GPT-2
 * lm-head of 64 or more rows is not among them).  Where it does, the two can differ where
 * logits tie to within rounding.  workspace is
 * device memory of at least matmul_forward_argmax_workspace(B, T, OC) bytes.  Other shapes
 * take a slow one-block-per-row kernel and ignore the workspace.  No counterpart in the
 * reference, which runs its matmul launcher (kernels/matmul/2_matmul_cublas.cuh:34) and
 * reads all logits back. */
size_t matmul_forward_argmax_workspace(int B, int T, int OC);
int matmul_forward_argmax_status(int* ids, void* workspace, size_t workspace_bytes, const float* inp,
                                 const float* weight, const float* bias, int B, int T, int C,
                                 int OC);

/* matmul_forward_argmax for callers that cannot allocate or hand over a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The (value, column) pairs go to a static array of
 * GPT2HIP_ARGMAX_NOALLOC_BYTES bytes of device memory inside the library (every GPU the
 * library runs on holds it until the process ends); the call allocates and frees nothing.
 * Shapes whose pairs need more (matmul_forward_argmax_workspace(B, T, OC) bytes; the limit
 * covers B*T = 8192 rows at OC = 50257..50304) are rejected with GPT2HIP_EINVAL.  Results equal
 * matmul_forward_argmax_status bit for bit.  All calls on one GPU share the array: calls
 * that overlap on one GPU (different streams or threads) race.  The first call on a device
 * looks the array's address up (no allocation, but make it outside graph capture). */
#define GPT2HIP_ARGMAX_NOALLOC_BYTES (33u << 20)
int matmul_forward_argmax_noalloc_status(int* ids, const float* inp, const float* weight,
                                         const float* bias, int B, int T, int C, int OC);

/* ---- whole model: the gpt2_forward driver (llm.c train_gpt2_fp32.cu's
 * gpt2_forward, which the reference plugs its kernels into, README.md:19;
 * dataflow in reference images/gpt2/gpt2_flow.png). ---- */

typedef struct {
  int max_seq_len; /* maxT */
  int vocab_size;  /* V    */
  int num_layers;  /* L    */
  int num_heads;   /* NH   */
  int channels;    /* C    */
} GPT2Config;

typedef struct GPT2 GPT2; /* opaque */

/* Allocates the parameter buffer (uninitialised) on the current device.
 * Returns NULL on failure (see gpt2hip_last_error). */
GPT2* gpt2_create(const GPT2Config* config);
void gpt2_destroy(GPT2* model);

/* Number of fp32 parameters, and the flat device buffer that holds them in
 * llm.c checkpoint order: wte(V,C) wpe(maxT,C) ln1w(L,C) ln1b(L,C)
 * qkvw(L,3C,C) qkvb(L,3C) attprojw(L,C,C) attprojb(L,C) ln2w(L,C) ln2b(L,C)
 * fcw(L,4C,C) fcb(L,4C) fcprojw(L,C,4C) fcprojb(L,C) lnfw(C) lnfb(C). */
size_t gpt2_num_parameters(const GPT2* model);
float* gpt2_params_device(GPT2* model);
/* Copies n = gpt2_num_parameters floats from host memory into that buffer. */
int gpt2_load_params_host(GPT2* model, const float* host_params, size_t n);

/* llm.c checkpoint files (gpt2_124M.bin, gpt2_124M_bf16.bin): 256 int32 header words
 * {20240326, version, maxT, V, L, NH, C, padded V, ...} followed by the tensors in the
 * order above.  Version 3 (fp32) and version 5 (bf16, widened to fp32 on load, which is
 * exact) store wte with its rows padded to "padded V" (the pad rows are skipped on load:
 * this library keeps wte unpadded); version 1 (fp32) has no padding.  Other versions are
 * rejected.  gpt2_checkpoint_read_config touches no GPU.
 * gpt2_build_from_checkpoint mirrors llm.c's function of that name
 * (gpt2_build_from_checkpoint(GPT2*, const char*)); it returns NULL on failure. */
int gpt2_checkpoint_read_config(const char* path, GPT2Config* config);
GPT2* gpt2_build_from_checkpoint(const char* path);

/* Allocates activations for up to B*T tokens (forward does this on demand; call
 * it up front to keep allocation out of a timed region). */
int gpt2_reserve(GPT2* model, int B, int T);

/* Forward pass.  gpt2_forward takes HOST token ids like llm.c and copies them
 * in; gpt2_forward_device takes ids already on the device.  Afterwards
 * gpt2_logits() is (B,T,V) on the device.  Launches are asynchronous.  Host ids
 * outside [0, vocab_size) are rejected; device ids are checked by the first kernel,
 * which fills the rows of bad ids with NaN instead of reading outside the table. */
int gpt2_forward_status(GPT2* model, const int* inputs_host, int B, int T);
void gpt2_forward(GPT2* model, const int* inputs_host, int B, int T);
int gpt2_forward_device_status(GPT2* model, const int* inputs_device, int B, int T);
/* gpt2_forward_device replayed from a HIP graph: the first call for a (B, T) runs the pass
 * once eagerly, captures its launches and instantiates the graph; later calls copy the
 * ids in and launch the graph on the calling thread's stream.  The graphs are dropped
 * when a larger B*T makes the model reallocate its activations.  No counterpart in the
 * reference.  (At B=8, T=1024 the launches are not the bound and the graph gains nothing;
 * it is for short prompts, where the host would otherwise issue ~90 launches per ms.) */
int gpt2_forward_graph_status(GPT2* model, const int* inputs_device, int B, int T);
/* Incremental inference with a key/value cache (no counterpart in the reference, whose
 * driver only runs whole sequences).  gpt2_prefill runs a prompt of B sequences of T
 * tokens (ids on the device), stores every layer's keys and values in a cache sized for
 * max_seq_len positions, and computes the logits of the LAST position of each sequence
 * only.  gpt2_decode appends one token per sequence (B ids on the device) at the next
 * position: one row per sequence goes through the same launchers, attention reads the
 * cache.  After either call gpt2_step_logits() is (B, vocab_size) on the device and
 * gpt2_cache_length() the number of positions held; the step's logits equal the logits a
 * full forward pass over the extended sequences gives at that position (to fp32
 * rounding).  gpt2_logits() / gpt2_argmax_status() describe full passes only. */
int gpt2_prefill_status(GPT2* model, const int* inputs_device, int B, int T);
int gpt2_decode_status(GPT2* model, const int* next_ids_device);
/* How gpt2_decode runs (no counterpart in the reference).  persistent != 0 (the default): one
 * persistent kernel per step where it takes the model (up to 16 sequences, head size 64,
 * channels 256, 512, 768 or 1024, a device with at least 256 compute units), otherwise one
 * launch per operation; 0: always one launch per operation.  spin_limit bounds the polls a
 * workgroup of the persistent kernel spends on one flag of its grid barrier before it gives
 * up and ends the kernel (default 2^21).  A step that gave up leaves NaN in gpt2_step_logits(),
 * and so does every step already queued behind it (never stale values of an earlier step).
 * The failure is reported once, by the first of gpt2_decode_status (if the step has ended by
 * then: it never waits) or gpt2_decode_sync_status (which waits); by then the cache has been
 * rolled back to the positions before the failed step (gpt2_cache_length()), so decoding can
 * resume from there, and the model runs one launch per operation until gpt2_decode_options
 * asks for the persistent kernel again.  gpt2_prefill_status clears a failure nobody asked
 * about (it rebuilds the cache anyway).  gpt2_decode_options itself waits for the steps queued
 * so far and, if one of them gave up and nobody has been told yet, applies the new options and
 * then returns that failure (rolled-back cache as above) instead of 0. */
int gpt2_decode_options(GPT2* model, int persistent, unsigned spin_limit);
/* Waits until every decode step queued so far has ended and reports whether one of the
 * persistent kernel's steps gave up (see gpt2_decode_options); 0 if all of them completed.
 * Call it before trusting ids or logits produced by steps that were queued without
 * synchronisation.  No counterpart in the reference. */
int gpt2_decode_sync_status(GPT2* model);
/* One gpt2_decode step of the persistent kernel with a clock probe: every workgroup g records
 * the 100 MHz wall clock when it has finished the work of phase p (clocks[(2p) * G + g]) and
 * when it has passed the grid barrier after it (clocks[(2p + 1) * G + g]); phases are, per
 * layer, qkv GEMM, attention, projection GEMM, fc GEMM, fc projection GEMM, then the lm-head
 * (work only).  G = 256, the kernel's workgroups; gpt2_decode_probe_size() = the slots needed
 * (0 if the persistent kernel does not take the model at the prefilled batch size). */
int gpt2_decode_probe_status(GPT2* model, const int* next_ids_device, unsigned long long* clocks_device,
                             size_t capacity);
size_t gpt2_decode_probe_size(const GPT2* model);
const float* gpt2_step_logits(const GPT2* model);
int gpt2_cache_length(const GPT2* model);

/* Whether gpt2_forward at this size forms the two residual sums of a block in the epilogues of
 * the projections (matmul_forward_residual_status, followed by layernorm_forward on the sum)
 * rather than in fused_residual_layernorm_forward: 1 from B*T*channels = 3 000 000 on, where it
 * is the faster of the two; the logits are the same bit for bit either way.  In the profiled
 * pass GPT2_PROF_FUSED_RESIDUAL_LAYERNORM then holds those layernorm_forward launches and the two
 * projections' categories include the add.  Touches no GPU. */
int gpt2_forward_sums_in_matmul(const GPT2Config* config, int B, int T);

/* Forward pass that keeps only the argmax of every position's logits (greedy next
 * token ids, B*T ints on the device): the lm-head runs as matmul_forward_argmax, the
 * logits buffer is not written and gpt2_argmax_status is unavailable afterwards. */
int gpt2_forward_argmax_status(GPT2* model, const int* inputs_device, int B, int T,
                               int* next_ids_device);
/* The same forward pass with a HIP event recorded on the null stream around
 * every launch; waits for completion and adds each launch's elapsed ms into
 * ms_per_category[GPT2_PROF_COUNT] (host memory).  No counterpart in the
 * reference, whose timings come from an external profiler (README.md:179). */
enum {
  GPT2_PROF_ENCODER = 0,
  GPT2_PROF_LAYERNORM,
  GPT2_PROF_MATMUL_QKV,
  GPT2_PROF_ATTENTION,
  GPT2_PROF_MATMUL_ATTPROJ,
  GPT2_PROF_FUSED_RESIDUAL_LAYERNORM,
  GPT2_PROF_MATMUL_FC_GELU,
  GPT2_PROF_MATMUL_FCPROJ,
  GPT2_PROF_MATMUL_LMHEAD,
  GPT2_PROF_COUNT
};
int gpt2_forward_profiled_status(GPT2* model, const int* inputs_device, int B, int T,
                                 float* ms_per_category);
/* What the event that gpt2_forward_profiled_status records after a launch adds to the
 * interval it closes, in microseconds: `launches` launches that do next to nothing, timed with
 * an event after each one and again back to back, difference per launch.  Allocates and frees
 * 1 KiB of device memory and waits for its launches; negative on failure.  For reading the
 * per-category times of short kernels (a diagnostic, like the profiled pass itself). */
float gpt2hip_profile_marker_overhead_us(int launches);
const float* gpt2_logits(const GPT2* model);
/* Final layernorm output (B,T,C) of the last forward, on the device. */
const float* gpt2_lnf(const GPT2* model);
/* Per-position argmax of the last forward's logits into ids_device (B*T). */
int gpt2_argmax_status(GPT2* model, int* ids_device);

/* The HIP stream (a hipStream_t) that every launcher, copy and timer of the calling
 * thread uses from now on; NULL, the initial value, is the null stream.  llm.c launches
 * on the null stream throughout (train_gpt2_fp32.cu), which is therefore the default. */
void gpt2hip_set_stream(void* hip_stream);
void* gpt2hip_get_stream(void);

/* A K-split workspace for the launchers that keep llm.c's signatures.  matmul_forward(out,
 * inp, weight, bias, B, T, C, OC) (reference kernels/matmul/2_matmul_cublas.cuh:34-42) and
 * matmul_forward_gelu (kernels/matmul/9_matmul_async_cg_tf32_gelu.cuh:237-246) have no
 * argument through which a caller could lend one; a caller that sets one here gets, from
 * those two launchers on the calling thread, exactly what matmul_forward_splitk_status gives
 * with the same workspace (same plan, same bits).  Same contract as there: device memory,
 * 256-byte aligned, the first GPT2HIP_SPLITK_COUNTER_BYTES zeroed once before the first use,
 * and ONE workspace per set of launches that may overlap on the GPU -- two threads, or two
 * streams of one thread, must not share one.  NULL / 0, the initial value, means none: the
 * launchers then choose a tile shape only.  The library's own gpt2_forward driver uses a
 * workspace that the model owns and ignores this setting.  Returns GPT2HIP_EINVAL for a
 * misaligned pointer or a size below the counters'. */
int gpt2hip_set_workspace(void* workspace, size_t workspace_bytes);

/* Event timer on the calling thread's stream (the stream its launchers use). */
typedef struct GPT2Timer GPT2Timer;
GPT2Timer* gpt2hip_timer_create(void);
void gpt2hip_timer_destroy(GPT2Timer* t);
int gpt2hip_timer_start(GPT2Timer* t);
/* Records the stop event, waits for it, returns elapsed ms (negative on error). */
float gpt2hip_timer_stop_ms(GPT2Timer* t);

#ifdef __cplusplus
}
#endif
#endif /* GPT2_MI355X_H */
