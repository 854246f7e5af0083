// Host side: the gpt2_forward driver, error string and event timer.
//
// gpt2_forward sequences the launchers the way llm.c's train_gpt2_fp32.cu does
// (reference README.md:9-19, images/gpt2/gpt2_flow.png), with the two fusions
// the reference introduces: residual+layernorm in one kernel (README.md:255-268)
// and GELU in the fc GEMM's epilogue (9_matmul_async_cg_tf32_gelu.cuh:196-212).
// Per layer: qkv GEMM, attention, projection GEMM, fused residual+layernorm,
// fc GEMM (+GELU), projection GEMM, fused residual+layernorm (whose layernorm
// is the NEXT layer's ln1, or the final layernorm after the last layer).
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <vector>

#include <dlfcn.h>

#include "common.hpp"

namespace g2 {

hipStream_t& stream_slot() {
  static thread_local hipStream_t s = nullptr;
  return s;
}

ThreadWorkspace& workspace_slot() {
  static thread_local ThreadWorkspace w;
  return w;
}

char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

enum { P_WTE, P_WPE, P_LN1W, P_LN1B, P_QKVW, P_QKVB, P_ATTPROJW, P_ATTPROJB, P_LN2W, P_LN2B,
       P_FCW, P_FCB, P_FCPROJW, P_FCPROJB, P_LNFW, P_LNFB, P_COUNT };

}  // namespace g2

struct GPT2 {
  GPT2Config cfg;
  int device;
  size_t num_params;
  size_t param_off[g2::P_COUNT];
  float* params;  // flat device buffer, checkpoint order

  // activations, sized for cap_tokens = B*T
  long long cap_tokens;
  int* ids;        // (M)
  float* res_a;    // (M,C) residual stream, ping
  float* res_b;    // (M,C) residual stream, pong
  float* ln;       // (M,C) layernorm output feeding the next GEMM
  float* qkv;      // (M,3C)
  float* atty;     // (M,C)
  float* proj;     // (M,C) attproj / fcproj output
  float* fch;      // (M,4C) gelu(fc)
  float* logits;   // (M,V)
  void* pairs;     // workspace of matmul_forward_argmax for (M,V)
  size_t pairs_bytes;
  void* splitk;    // workspace of matmul_forward_splitk: counters (zero between calls) + partial tiles
  size_t splitk_bytes;
  bool splitk_dirty;  // a pass that lent the workspace to its GEMMs did not get to its end
  int last_B, last_T;
  bool last_has_logits;

  // key/value cache of the incremental (prefill + decode) path: (L, 2, kv_batch, NH, maxT, hs),
  // and the logits of the newest position, (kv_batch, V)
  float* kv;
  float* step_logits;
  int kv_batch;  // sequences the cache is allocated for
  int kv_len;    // positions filled so far (the same for every sequence); 0 = empty

  // the persistent decode-step kernel: barrier flags + error word on the device, the epoch
  // its last launch ended with, a pinned host word that a step which gives up writes the
  // error into (looked at on the next call, once the event behind the step has passed)
  unsigned* step_flags;
  float* step_act;  // the activations it hands between workgroups (decode_step_activation_floats)
  unsigned step_epoch;
  unsigned* step_error_host;
  unsigned* step_error_device;  // the same pinned word as the device addresses it
  hipStream_t step_stream;   // the stream of the newest step
  bool step_pending;         // steps have been launched that nobody has waited for yet
  bool step_fallback;        // a step of the persistent kernel gave up: one launch per operation from then on
  bool step_persistent;      // use the persistent kernel where it takes the model
  unsigned step_spin_limit;  // polls of a barrier flag before a workgroup gives up

  // forward passes captured as HIP graphs, one per (B, T); they hold the activation
  // pointers, so they are dropped whenever the activations are reallocated
  struct Captured {
    int B, T;
    hipGraph_t graph;
    hipGraphExec_t exec;
  };
  std::vector<Captured> graphs;
};

namespace g2 {

static void drop_graphs(GPT2* m) {
  for (auto& g : m->graphs) {
    (void)hipGraphExecDestroy(g.exec);
    (void)hipGraphDestroy(g.graph);
  }
  m->graphs.clear();
}

static void free_activations(GPT2* m) {
  drop_graphs(m);
  void* ptrs[] = {m->ids,  m->res_a, m->res_b, m->ln,     m->qkv,
                  m->atty, m->proj,  m->fch,   m->logits, m->pairs, m->splitk};
  for (void* p : ptrs)
    if (p) (void)hipFree(p);
  m->ids = nullptr;
  m->res_a = m->res_b = m->ln = m->qkv = m->atty = m->proj = m->fch = m->logits = nullptr;
  m->pairs = m->splitk = nullptr;
  m->pairs_bytes = m->splitk_bytes = 0;
  m->cap_tokens = 0;
}

static void free_cache(GPT2* m) {
  if (m->kv) (void)hipFree(m->kv);
  if (m->step_logits) (void)hipFree(m->step_logits);
  if (m->step_flags) (void)hipFree(m->step_flags);
  if (m->step_act) (void)hipFree(m->step_act);
  m->step_act = nullptr;
  if (m->step_error_host) (void)hipHostFree(m->step_error_host);
  m->step_stream = nullptr;
  m->step_pending = false;
  m->kv = m->step_logits = nullptr;
  m->step_flags = m->step_error_host = m->step_error_device = nullptr;
  m->step_epoch = 0;
  m->kv_batch = m->kv_len = 0;
}

// Key/value cache and step logits for B sequences of up to max_seq_len positions.
static int reserve_cache(GPT2* m, int B) {
  if (B <= m->kv_batch) return GPT2HIP_OK;
  free_cache(m);
  const GPT2Config& c = m->cfg;
  const size_t kv_bytes = (size_t)c.num_layers * 2 * B * c.max_seq_len * c.channels * sizeof(float);
  hipError_t e = hipMalloc((void**)&m->kv, kv_bytes);
  if (e == hipSuccess) e = hipMalloc((void**)&m->step_logits, (size_t)B * c.vocab_size * sizeof(float));
  const size_t flag_bytes = decode_step_flag_bytes(m->device);
  if (e == hipSuccess && flag_bytes) e = hipMalloc((void**)&m->step_flags, flag_bytes);
  if (e == hipSuccess && flag_bytes) e = hipMemset(m->step_flags, 0, flag_bytes);
  // rows of sequences that do not exist are read (and ignored) by the kernel: keep them finite
  const size_t act_bytes = decode_step_activation_floats(c) * sizeof(float);
  if (e == hipSuccess) e = hipMalloc((void**)&m->step_act, act_bytes);
  if (e == hipSuccess) e = hipMemset(m->step_act, 0, act_bytes);
  if (e == hipSuccess) e = hipHostMalloc((void**)&m->step_error_host, sizeof(unsigned), hipHostMallocDefault);
  if (e == hipSuccess) *m->step_error_host = 0;
  if (e == hipSuccess) e = hipHostGetDevicePointer((void**)&m->step_error_device, m->step_error_host, 0);
  if (e != hipSuccess) {
    free_cache(m);
    return fail(GPT2HIP_ENOMEM, "gpt2: key/value cache for %d sequences (%zu bytes): %s", B, kv_bytes,
                hipGetErrorString(e));
  }
  m->kv_batch = B;
  return GPT2HIP_OK;
}

// The K-split counters are zero between GEMMs that ran to their end.  A pass that returned
// early (a failed launch) may have left a GEMM in between: the next pass clears them first.
static int begin_splitk_use(GPT2* m) {
  if (m->splitk_dirty && m->splitk)
    G2_HIP(hipMemsetAsync(m->splitk, 0, GPT2HIP_SPLITK_COUNTER_BYTES, stream()));
  m->splitk_dirty = true;
  return GPT2HIP_OK;
}

static int check_shape(const GPT2* m, int B, int T) {
  if (!m) return fail(GPT2HIP_EINVAL, "gpt2: null model");
  if (B < 1 || T < 1 || T > m->cfg.max_seq_len)
    return fail(GPT2HIP_EINVAL, "gpt2: bad B=%d T=%d (max_seq_len %d)", B, T, m->cfg.max_seq_len);
  if ((long long)B * T > (1LL << 24)) return fail(GPT2HIP_EINVAL, "gpt2: B*T=%lld too large", (long long)B * T);
  return GPT2HIP_OK;
}

static int reserve(GPT2* m, int B, int T) {
  if (int rc = check_shape(m, B, T)) return rc;
  const long long M = (long long)B * T;
  if (M <= m->cap_tokens) return GPT2HIP_OK;
  free_activations(m);
  const size_t C = m->cfg.channels, V = m->cfg.vocab_size, n = (size_t)M;
  struct { void** p; size_t bytes; } want[] = {
      {(void**)&m->ids, n * sizeof(int)},          {(void**)&m->res_a, n * C * 4},
      {(void**)&m->res_b, n * C * 4},              {(void**)&m->ln, n * C * 4},
      {(void**)&m->qkv, n * 3 * C * 4},            {(void**)&m->atty, n * C * 4},
      {(void**)&m->proj, n * C * 4},               {(void**)&m->fch, n * 4 * C * 4},
      {(void**)&m->logits, n * V * 4},
      {&m->pairs, matmul_forward_argmax_workspace(1, (int)M, (int)V)},
      {&m->splitk, matmul_forward_splitk_workspace()}};
  for (auto& w : want) {
    hipError_t e = hipMalloc(w.p, w.bytes);
    if (e != hipSuccess) {
      *w.p = nullptr;
      free_activations(m);
      return fail(GPT2HIP_ENOMEM, "gpt2: hipMalloc of %zu bytes failed: %s", w.bytes,
                  hipGetErrorString(e));
    }
  }
  m->pairs_bytes = matmul_forward_argmax_workspace(1, (int)M, (int)V);
  // the counters start at zero; every GEMM that uses them leaves them at zero
  if (hipMemset(m->splitk, 0, GPT2HIP_SPLITK_COUNTER_BYTES) != hipSuccess) {
    free_activations(m);
    return fail(GPT2HIP_EHIP, "gpt2: clearing the K-split counters failed");
  }
  m->splitk_bytes = matmul_forward_splitk_workspace();
  m->cap_tokens = M;
  return GPT2HIP_OK;
}

// Optional per-launch timing: an event is recorded on the null stream before the
// first launch and after every launch; category[i] names the launch between
// events i and i+1.
// Named ranges around the launches of the profiled forward pass, for a rocprofv3 marker
// trace (the counterpart of the reference's NVTX ranges, kernels/attention/
// 1_attention_cublas.cuh:44-67).  The marker library is looked up at run time, once: without
// it (or outside a profiler) the ranges are no-ops, and the timed entry points never touch it.
struct Roctx {
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
  Roctx() {
    void* h = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_LOCAL);
    if (!h) h = dlopen("librocprofiler-sdk-roctx.so.1", RTLD_NOW | RTLD_LOCAL);
    if (!h) return;
    push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
    pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
    if (!push || !pop) push = nullptr, pop = nullptr;
  }
};
static const Roctx& roctx() {
  static const Roctx r;  // thread-safe initialisation
  return r;
}
static const char* const kProfNames[GPT2_PROF_COUNT] = {
    "encoder_forward",       "layernorm_forward",
    "matmul_forward qkv",    "attention_forward",
    "matmul_forward attproj", "fused_residual_layernorm_forward",
    "matmul_forward_gelu fc", "matmul_forward fcproj",
    "matmul_forward lm-head"};

struct Profile {
  std::vector<hipEvent_t> events;  // the first `used` of them have been recorded
  std::vector<int> category;
  size_t used = 0;
  int reserve(size_t n) {
    while (events.size() < n) {
      hipEvent_t e;
      G2_HIP(hipEventCreate(&e));
      events.push_back(e);
    }
    return GPT2HIP_OK;
  }
  int mark(int cat) {  // cat < 0: the opening event
    if (int rc = reserve(used + 1)) return rc;
    if (cat >= 0) category.push_back(cat);
    G2_HIP(hipEventRecord(events[used++], stream()));
    return GPT2HIP_OK;
  }
  ~Profile() {
    for (hipEvent_t e : events) (void)hipEventDestroy(e);
  }
};

// The forward pass proper; ids are already in m->ids.  With next_ids the lm-head keeps
// only the argmax of every row (written there) and m->logits is left untouched.  With
// fill_cache (a prompt: the cache must hold B sequences) every layer's keys and values
// are also copied into the cache and the lm-head runs on the last position of each
// sequence only, into m->step_logits.
static int forward_resident(GPT2* m, int B, int T, Profile* prof = nullptr,
                            int* next_ids = nullptr, bool fill_cache = false) {
  const GPT2Config& c = m->cfg;
  const int C = c.channels, L = c.num_layers, NH = c.num_heads, V = c.vocab_size;
  const size_t cs = (size_t)C;
  auto P = [&](int which) { return m->params + m->param_off[which]; };
#define G2_TRY(call)                  \
  do {                                \
    if (int rc_ = (call)) return rc_; \
  } while (0)
#define G2_STEP(cat, call)                                   \
  do {                                                       \
    if (prof && roctx().push) roctx().push(kProfNames[cat]); \
    const int rc_step_ = (call);                             \
    if (prof && roctx().pop) roctx().pop();                  \
    if (rc_step_) return rc_step_;                           \
    if (prof) G2_TRY(prof->mark(cat));                       \
  } while (0)
  G2_TRY(begin_splitk_use(m));
  if (prof) G2_TRY(prof->mark(-1));

  float* residual = m->res_a;  // current residual stream
  float* other = m->res_b;
  // Where the two residual adds of a block happen.  The reference adds in the kernel that also
  // normalises (fused_residual_layernorm_forward: one pass reads the stream and the update and
  // writes the sum and its normalisation); from a few thousand rows on the pass pays to add in
  // the projection's epilogue instead (matmul_forward_residual_status) and to normalise the sum
  // by layernorm_forward, which moves half the bytes -- the same additions, bit for bit.
  const bool sum_in_matmul = gpt2_forward_sums_in_matmul(&c, B, T) != 0;
  G2_STEP(GPT2_PROF_ENCODER, encoder_launch(residual, m->ids, P(P_WTE), P(P_WPE), B, T, C, V));
  // the one stand-alone layernorm: ln1 of layer 0
  G2_STEP(GPT2_PROF_LAYERNORM, layernorm_forward_status(m->ln, nullptr, nullptr, residual, P(P_LN1W), P(P_LN1B), B, T, C));
  // The four GEMMs of a block may split K between workgroups through the model's workspace
  // (short prompts, where a layer has fewer tiles than the device has compute units).
  for (int l = 0; l < L; l++) {
    G2_STEP(GPT2_PROF_MATMUL_QKV, matmul_forward_splitk_status(m->qkv, m->ln, P(P_QKVW) + l * 3 * cs * cs, P(P_QKVB) + l * 3 * cs,
                                 B, T, C, 3 * C, 0, m->splitk, m->splitk_bytes));
    if (fill_cache) {
      const size_t plane = (size_t)m->kv_batch * c.max_seq_len * cs;
      G2_TRY(kv_store_launch(m->kv + (2 * (size_t)l) * plane, m->kv + (2 * (size_t)l + 1) * plane, m->qkv,
                             B, T, c.max_seq_len, C, NH));
    }
    G2_STEP(GPT2_PROF_ATTENTION, attention_forward_status(m->atty, nullptr, nullptr, m->qkv, B, T, C, NH));
    // residual2 = residual + attproj ; ln = ln2(residual2)
    if (sum_in_matmul) {
      G2_STEP(GPT2_PROF_MATMUL_ATTPROJ, matmul_forward_residual_status(other, m->atty, P(P_ATTPROJW) + l * cs * cs,
                                   P(P_ATTPROJB) + l * cs, residual, B, T, C, C, m->splitk, m->splitk_bytes));
      G2_STEP(GPT2_PROF_FUSED_RESIDUAL_LAYERNORM, layernorm_forward_status(m->ln, nullptr, nullptr, other, P(P_LN2W) + l * cs,
                                   P(P_LN2B) + l * cs, B, T, C));
    } else {
      G2_STEP(GPT2_PROF_MATMUL_ATTPROJ, matmul_forward_splitk_status(m->proj, m->atty, P(P_ATTPROJW) + l * cs * cs,
                                   P(P_ATTPROJB) + l * cs, B, T, C, C, 0, m->splitk, m->splitk_bytes));
      G2_STEP(GPT2_PROF_FUSED_RESIDUAL_LAYERNORM, fused_residual_layernorm_forward_status(other, m->ln, nullptr, nullptr, residual,
                                                     m->proj, P(P_LN2W) + l * cs, P(P_LN2B) + l * cs,
                                                     B, T, C));
    }
    G2_STEP(GPT2_PROF_MATMUL_FC_GELU, matmul_forward_splitk_status(m->fch, m->ln, P(P_FCW) + l * 4 * cs * cs,
                                      P(P_FCB) + l * 4 * cs, B, T, C, 4 * C, 1, m->splitk, m->splitk_bytes));
    // residual3 = residual2 + fcproj ; ln = ln1 of the next layer, or the final layernorm
    const float* nw = (l + 1 < L) ? P(P_LN1W) + (l + 1) * cs : P(P_LNFW);
    const float* nb = (l + 1 < L) ? P(P_LN1B) + (l + 1) * cs : P(P_LNFB);
    if (sum_in_matmul) {
      G2_STEP(GPT2_PROF_MATMUL_FCPROJ, matmul_forward_residual_status(residual, m->fch, P(P_FCPROJW) + l * 4 * cs * cs,
                                   P(P_FCPROJB) + l * cs, other, B, T, 4 * C, C, m->splitk, m->splitk_bytes));
      G2_STEP(GPT2_PROF_FUSED_RESIDUAL_LAYERNORM, layernorm_forward_status(m->ln, nullptr, nullptr, residual, nw, nb, B, T, C));
    } else {
      G2_STEP(GPT2_PROF_MATMUL_FCPROJ, matmul_forward_splitk_status(m->proj, m->fch, P(P_FCPROJW) + l * 4 * cs * cs,
                                   P(P_FCPROJB) + l * cs, B, T, 4 * C, C, 0, m->splitk, m->splitk_bytes));
      G2_STEP(GPT2_PROF_FUSED_RESIDUAL_LAYERNORM, fused_residual_layernorm_forward_status(residual, m->ln, nullptr, nullptr, other,
                                                     m->proj, nw, nb, B, T, C));
    }
  }
  // lm-head: weight-tied to wte, no bias, unpadded vocabulary
  if (fill_cache) {
    // rows (b, T-1) of the final layernorm, gathered into the first B rows of m->atty
    G2_HIP(hipMemcpy2DAsync(m->atty, cs * 4, m->ln + (size_t)(T - 1) * cs, (size_t)T * cs * 4, cs * 4, B,
                            hipMemcpyDeviceToDevice, stream()));
    G2_TRY(matmul_forward_splitk_status(m->step_logits, m->atty, P(P_WTE), nullptr, B, 1, C, V, 0, m->splitk,
                                        m->splitk_bytes));
  } else if (next_ids)
    G2_STEP(GPT2_PROF_MATMUL_LMHEAD, matmul_forward_argmax_status(next_ids, m->pairs, m->pairs_bytes, m->ln,
                                                                  P(P_WTE), nullptr, B, T, C, V));
  else
    G2_STEP(GPT2_PROF_MATMUL_LMHEAD, matmul_forward_splitk_status(m->logits, m->ln, P(P_WTE), nullptr, B, T, C, V, 0,
                                                                  m->splitk, m->splitk_bytes));
#undef G2_STEP
#undef G2_TRY
  m->splitk_dirty = false;
  m->last_B = B;
  m->last_T = T;
  m->last_has_logits = next_ids == nullptr && !fill_cache;
  return GPT2HIP_OK;
}

}  // namespace g2

extern "C" {

const char* gpt2hip_last_error(void) { return g2::last_error_buffer(); }

void gpt2hip_set_stream(void* hip_stream) { g2::stream_slot() = static_cast<hipStream_t>(hip_stream); }
void* gpt2hip_get_stream(void) { return g2::stream_slot(); }

int gpt2hip_set_workspace(void* workspace, size_t workspace_bytes) {
  using namespace g2;
  if (!workspace || workspace_bytes == 0) {
    workspace_slot() = ThreadWorkspace{};
    return GPT2HIP_OK;
  }
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return fail(GPT2HIP_EINVAL, "gpt2hip_set_workspace: workspace must be 256-byte aligned");
  if (workspace_bytes < GPT2HIP_SPLITK_COUNTER_BYTES)
    return fail(GPT2HIP_EINVAL, "gpt2hip_set_workspace: %zu bytes do not hold the %u bytes of counters",
                workspace_bytes, GPT2HIP_SPLITK_COUNTER_BYTES);
  workspace_slot() = ThreadWorkspace{workspace, workspace_bytes};
  return GPT2HIP_OK;
}

GPT2* gpt2_create(const GPT2Config* config) {
  using namespace g2;
  if (!config || config->max_seq_len < 1 || config->vocab_size < 1 || config->num_layers < 1 ||
      config->num_heads < 1 || config->channels < 1 || config->channels % config->num_heads != 0) {
    fail(GPT2HIP_EINVAL, "gpt2_create: invalid config");
    return nullptr;
  }
  GPT2* m = new GPT2();
  m->cfg = *config;
  m->step_persistent = true;
  m->step_spin_limit = 1u << 21;
  const size_t V = config->vocab_size, maxT = config->max_seq_len, L = config->num_layers,
               C = config->channels;
  const size_t sizes[P_COUNT] = {V * C,         maxT * C, L * C,         L * C,
                                 L * 3 * C * C, L * 3 * C, L * C * C,     L * C,
                                 L * C,         L * C,     L * 4 * C * C, L * 4 * C,
                                 L * C * 4 * C, L * C,     C,             C};
  size_t off = 0;
  for (int i = 0; i < P_COUNT; i++) {
    m->param_off[i] = off;
    off += sizes[i];
  }
  m->num_params = off;
  if (hipGetDevice(&m->device) != hipSuccess ||
      hipMalloc((void**)&m->params, off * sizeof(float)) != hipSuccess) {
    fail(GPT2HIP_ENOMEM, "gpt2_create: cannot allocate %zu parameter bytes", off * sizeof(float));
    delete m;
    return nullptr;
  }
  return m;
}

void gpt2_destroy(GPT2* model) {
  if (!model) return;
  g2::free_activations(model);
  g2::free_cache(model);
  if (model->params) (void)hipFree(model->params);
  delete model;
}

size_t gpt2_num_parameters(const GPT2* model) { return model ? model->num_params : 0; }
float* gpt2_params_device(GPT2* model) { return model ? model->params : nullptr; }

int gpt2_load_params_host(GPT2* model, const float* host_params, size_t n) {
  using namespace g2;
  if (!model || !host_params) return fail(GPT2HIP_EINVAL, "gpt2_load_params_host: null pointer");
  if (n != model->num_params)
    return fail(GPT2HIP_EINVAL, "gpt2_load_params_host: got %zu floats, model has %zu", n,
                model->num_params);
  G2_HIP(hipMemcpy(model->params, host_params, n * sizeof(float), hipMemcpyHostToDevice));
  return GPT2HIP_OK;
}

namespace g2 {

// Reads and validates the 256-word header; on success *padded_v is the number of wte
// rows stored in the file and *elem_bytes the size of a stored parameter: 4 (fp32, versions
// 1 and 3) or 2 (bf16, version 5, which widens to fp32 exactly).
static int read_checkpoint_header(FILE* f, const char* path, GPT2Config* cfg, int* padded_v,
                                  int* elem_bytes) {
  int header[256];
  if (fread(header, sizeof(int), 256, f) != 256)
    return fail(GPT2HIP_EINVAL, "checkpoint %s: shorter than its 1024-byte header", path);
  if (header[0] != 20240326)
    return fail(GPT2HIP_EINVAL, "checkpoint %s: bad magic %d (want 20240326)", path, header[0]);
  if (header[1] != 1 && header[1] != 3 && header[1] != 5)
    return fail(GPT2HIP_EINVAL, "checkpoint %s: version %d is neither an fp32 (1, 3) nor a bf16 (5) checkpoint",
                path, header[1]);
  *elem_bytes = header[1] == 5 ? 2 : 4;
  cfg->max_seq_len = header[2];
  cfg->vocab_size = header[3];
  cfg->num_layers = header[4];
  cfg->num_heads = header[5];
  cfg->channels = header[6];
  *padded_v = (header[1] == 1) ? header[3] : header[7];
  if (cfg->max_seq_len < 1 || cfg->vocab_size < 1 || cfg->num_layers < 1 || cfg->num_heads < 1 ||
      cfg->channels < 1 || cfg->channels % cfg->num_heads != 0 || *padded_v < cfg->vocab_size)
    return fail(GPT2HIP_EINVAL, "checkpoint %s: implausible header (maxT %d V %d L %d NH %d C %d Vp %d)",
                path, header[2], header[3], header[4], header[5], header[6], *padded_v);
  return GPT2HIP_OK;
}

}  // namespace g2

int gpt2_checkpoint_read_config(const char* path, GPT2Config* config) {
  using namespace g2;
  if (!path || !config) return fail(GPT2HIP_EINVAL, "gpt2_checkpoint_read_config: null pointer");
  FILE* f = fopen(path, "rb");
  if (!f) return fail(GPT2HIP_EINVAL, "cannot open checkpoint %s", path);
  int padded_v = 0, elem_bytes = 0;
  const int rc = read_checkpoint_header(f, path, config, &padded_v, &elem_bytes);
  fclose(f);
  return rc;
}

GPT2* gpt2_build_from_checkpoint(const char* path) {
  using namespace g2;
  if (!path) {
    fail(GPT2HIP_EINVAL, "gpt2_build_from_checkpoint: null path");
    return nullptr;
  }
  FILE* f = fopen(path, "rb");
  if (!f) {
    fail(GPT2HIP_EINVAL, "cannot open checkpoint %s", path);
    return nullptr;
  }
  GPT2Config cfg;
  int padded_v = 0, elem_bytes = 0;
  GPT2* m = nullptr;
  if (read_checkpoint_header(f, path, &cfg, &padded_v, &elem_bytes) == GPT2HIP_OK && (m = gpt2_create(&cfg))) {
    // Stream the file through a bounded host buffer; skip wte's pad rows.
    const size_t C = cfg.channels;
    const size_t chunk = 16u << 20;  // floats
    std::vector<float> buf(chunk);
    std::vector<unsigned short> half(elem_bytes == 2 ? chunk : 0);
    size_t done = 0;  // floats written to the device buffer
    bool ok = true;
    while (ok && done < m->num_params) {
      if (done == (size_t)cfg.vocab_size * C && padded_v > cfg.vocab_size)
        ok = fseek(f, (long)((size_t)(padded_v - cfg.vocab_size) * C * (size_t)elem_bytes), SEEK_CUR) == 0;
      // never read across the end of wte, so that the pad can be skipped exactly there
      size_t want = std::min(chunk, m->num_params - done);
      if (done < (size_t)cfg.vocab_size * C) want = std::min(want, (size_t)cfg.vocab_size * C - done);
      const size_t got = !ok ? 0
                         : elem_bytes == 2 ? fread(half.data(), 2, want, f)
                                           : fread(buf.data(), sizeof(float), want, f);
      if (ok && got != want) {
        fail(GPT2HIP_EINVAL, "checkpoint %s: truncated (needs %zu parameters)", path, m->num_params);
        ok = false;
      }
      if (ok && elem_bytes == 2) {
        // bf16 is the upper half of an fp32: widening is exact
        for (size_t i = 0; i < want; i++) {
          const unsigned bits = (unsigned)half[i] << 16;
          memcpy(&buf[i], &bits, sizeof(float));
        }
      }
      if (ok && hipMemcpy(m->params + done, buf.data(), want * sizeof(float),
                          hipMemcpyHostToDevice) != hipSuccess) {
        fail(GPT2HIP_EHIP, "checkpoint %s: copy to the device failed", path);
        ok = false;
      }
      done += want;
    }
    if (!ok) {
      gpt2_destroy(m);
      m = nullptr;
    }
  }
  fclose(f);
  return m;
}

int gpt2_reserve(GPT2* model, int B, int T) { return g2::reserve(model, B, T); }

int gpt2_forward_status(GPT2* model, const int* inputs_host, int B, int T) {
  using namespace g2;
  if (int rc = reserve(model, B, T)) return rc;
  if (!inputs_host) return fail(GPT2HIP_EINVAL, "gpt2_forward: null inputs");
  const size_t n = (size_t)B * T;
  for (size_t i = 0; i < n; i++)
    if (inputs_host[i] < 0 || inputs_host[i] >= model->cfg.vocab_size)
      return fail(GPT2HIP_EINVAL, "gpt2_forward: token id %d at position %zu outside [0,%d)",
                  inputs_host[i], i, model->cfg.vocab_size);
  // in stream order after the previous pass; the host buffer is free again on return
  G2_HIP(hipMemcpyAsync(model->ids, inputs_host, n * sizeof(int), hipMemcpyHostToDevice, stream()));
  G2_HIP(hipStreamSynchronize(stream()));
  return forward_resident(model, B, T);
}

void gpt2_forward(GPT2* model, const int* inputs_host, int B, int T) {
  if (gpt2_forward_status(model, inputs_host, B, T)) g2::die("gpt2_forward");
}

int gpt2_forward_device_status(GPT2* model, const int* inputs_device, int B, int T) {
  using namespace g2;
  if (int rc = reserve(model, B, T)) return rc;
  if (!inputs_device) return fail(GPT2HIP_EINVAL, "gpt2_forward_device: null inputs");
  G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                        hipMemcpyDeviceToDevice, stream()));
  return forward_resident(model, B, T);
}

int gpt2_forward_graph_status(GPT2* model, const int* inputs_device, int B, int T) {
  using namespace g2;
  if (int rc = reserve(model, B, T)) return rc;  // drops the captured graphs if it reallocates
  if (!inputs_device) return fail(GPT2HIP_EINVAL, "gpt2_forward_graph: null inputs");
  GPT2::Captured* hit = nullptr;
  for (auto& g : model->graphs)
    if (g.B == B && g.T == T) hit = &g;
  if (!hit) {
    // One eager pass first: it raises the kernels' LDS limits, which is not stream work
    // and stays out of the capture.  Then the same launches are recorded from a stream
    // of their own (default priority) and instantiated.
    G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                          hipMemcpyDeviceToDevice, stream()));
    if (int rc = forward_resident(model, B, T)) return rc;
    G2_HIP(hipStreamSynchronize(stream()));
    hipStream_t cap = nullptr;
    G2_HIP(hipStreamCreateWithFlags(&cap, hipStreamNonBlocking));
    hipStream_t const caller = stream_slot();
    stream_slot() = cap;
    hipError_t e = hipStreamBeginCapture(cap, hipStreamCaptureModeThreadLocal);
    int rc = GPT2HIP_OK;
    hipGraph_t graph = nullptr;
    if (e == hipSuccess) {
      rc = forward_resident(model, B, T);
      e = hipStreamEndCapture(cap, &graph);  // also ends a capture that a failed launch broke
    }
    stream_slot() = caller;
    (void)hipStreamDestroy(cap);
    if (rc) {
      if (graph) (void)hipGraphDestroy(graph);
      return rc;
    }
    if (e != hipSuccess || !graph)
      return fail(GPT2HIP_EHIP, "gpt2_forward_graph: capture failed: %s", hipGetErrorString(e));
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
      (void)hipGraphDestroy(graph);
      return fail(GPT2HIP_EHIP, "gpt2_forward_graph: hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    model->graphs.push_back({B, T, graph, exec});
    hit = &model->graphs.back();
  }
  G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                        hipMemcpyDeviceToDevice, stream()));
  G2_HIP(hipGraphLaunch(hit->exec, stream()));
  model->last_B = B;
  model->last_T = T;
  model->last_has_logits = true;
  return GPT2HIP_OK;
}

int gpt2_forward_sums_in_matmul(const GPT2Config* config, int B, int T) {
  // Measured on GPT-2 124M / 350M at T = 1024: with the sum formed in the projections a pass takes
  // 1.0 % less at B = 8 and at B = 4 (the normalisation kernel 8.7 us less per launch at B*T =
  // 8192, the projection 1 us more), the same at B = 2, and 2 % more at B*T = 256, where both
  // kernels are bound by their launch and the projection's epilogue waits for its reads.
  return config && (long long)B * T * config->channels >= 3000000LL;
}

namespace g2 {
// Looks at the error word of the persistent decode-step kernel once the copy behind the
// newest step has arrived (wait: block until it has; otherwise only if it already has).  A
// step that gave up a barrier wait left NaN logits, and so did every step queued behind it;
// the word names its position.  Recovery: the cache is rolled back to the positions before
// that step, the barrier state is cleared, and the model decodes with one launch per
// operation from then on.  Returns an error exactly once per failure.
static int settle_steps(GPT2* m, bool wait) {
  if (!m->step_pending) return GPT2HIP_OK;
  // The workgroup that gives up writes the pinned word itself (system scope), so a look at it
  // costs nothing and needs no event behind every step; only a caller that wants to be sure that
  // every queued step has ended waits, for the stream the steps were queued on.
  if (wait) {
    G2_HIP(hipStreamSynchronize(m->step_stream));
    m->step_pending = false;
  }
  const unsigned word = __atomic_load_n(m->step_error_host, __ATOMIC_ACQUIRE);
  if (word == 0) return GPT2HIP_OK;
  *m->step_error_host = 0;
  G2_HIP(hipMemsetAsync(m->step_flags, 0, decode_step_flag_bytes(m->device), m->step_stream));
  m->step_epoch = 0;
  m->step_fallback = true;
  const int failed = (int)word - 1;
  if (m->kv_len > failed) m->kv_len = failed;
  return fail(GPT2HIP_EHIP,
              "gpt2_decode: the step at position %d gave up waiting at a grid barrier; its logits and "
              "those of the steps queued behind it are NaN, the cache is rolled back to %d positions "
              "and further steps run one launch per operation", failed, m->kv_len);
}
}  // namespace g2

int gpt2_decode_sync_status(GPT2* model) {
  if (!model) return g2::fail(GPT2HIP_EINVAL, "gpt2_decode_sync: null model");
  return g2::settle_steps(model, true);
}

int gpt2_prefill_status(GPT2* model, const int* inputs_device, int B, int T) {
  using namespace g2;
  if (!model) return fail(GPT2HIP_EINVAL, "gpt2_prefill: null model");
  // a failure among earlier decode steps that nobody has asked about: the cache is rebuilt
  // here anyway, so only the recovery (cleared barrier state, launch-per-operation steps) matters
  if (settle_steps(model, true)) last_error_buffer()[0] = 0;  // not this call's failure
  if (int rc = reserve(model, B, T)) return rc;
  if (!inputs_device) return fail(GPT2HIP_EINVAL, "gpt2_prefill: null inputs");
  if (model->kv_batch != B) {  // the cache planes are indexed with the batch it was sized for
    free_cache(model);
    if (int rc = reserve_cache(model, B)) return rc;
  }
  model->kv_len = 0;
  G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                        hipMemcpyDeviceToDevice, stream()));
  if (int rc = forward_resident(model, B, T, nullptr, nullptr, true)) return rc;
  model->kv_len = T;
  return GPT2HIP_OK;
}

namespace g2 {
static int decode_step(GPT2* model, const int* next_ids_device, unsigned long long* trace);
}

int gpt2_decode_status(GPT2* model, const int* next_ids_device) {
  return g2::decode_step(model, next_ids_device, nullptr);
}

int gpt2_decode_probe_status(GPT2* model, const int* next_ids_device, unsigned long long* clocks_device,
                             size_t capacity) {
  using namespace g2;
  if (!model || !clocks_device) return fail(GPT2HIP_EINVAL, "gpt2_decode_probe: null pointer");
  const size_t need = gpt2_decode_probe_size(model);
  if (need == 0)
    return fail(GPT2HIP_EINVAL, "gpt2_decode_probe: the persistent kernel does not take this model");
  if (capacity < need)
    return fail(GPT2HIP_EINVAL, "gpt2_decode_probe: %zu clock slots given, %zu needed", capacity, need);
  return decode_step(model, next_ids_device, clocks_device);
}

size_t gpt2_decode_probe_size(const GPT2* model) {
  using namespace g2;
  if (!model || !model->step_persistent || model->step_fallback || model->kv_batch < 1 ||
      !decode_step_supported(model->cfg, model->kv_batch, model->device))
    return 0;
  return decode_step_probe_slots(model->cfg.num_layers);
}

namespace g2 {
static int decode_step(GPT2* model, const int* next_ids_device, unsigned long long* trace) {
  if (!model || !next_ids_device) return fail(GPT2HIP_EINVAL, "gpt2_decode: null pointer");
  GPT2* m = model;
  const GPT2Config& c = m->cfg;
  // what is already known about earlier steps (never waits: steps are queued without
  // synchronisation; a failure not yet visible here turns this step's logits into NaN too)
  if (int rc = settle_steps(m, false)) return rc;
  if (m->kv_len < 1) return fail(GPT2HIP_EINVAL, "gpt2_decode: no prompt has been prefilled");
  if (m->kv_len >= c.max_seq_len)
    return fail(GPT2HIP_EINVAL, "gpt2_decode: the cache is full (%d positions)", c.max_seq_len);
  const int B = m->kv_batch, pos = m->kv_len;
  const int C = c.channels, L = c.num_layers, NH = c.num_heads, V = c.vocab_size;
  const size_t cs = (size_t)C;
  auto P = [&](int which) { return m->params + m->param_off[which]; };
#define G2_TRY(call)                  \
  do {                                \
    if (int rc_ = (call)) return rc_; \
  } while (0)
  // One row per sequence; the activation buffers of the prompt (sized for B*T >= B rows)
  // are reused.
  float* residual = m->res_a;
  float* other = m->res_b;
  const bool persistent = m->step_persistent && !m->step_fallback && m->step_flags && m->step_act &&
                          decode_step_supported(c, B, m->device);
  if (!persistent)  // the persistent kernel gathers the embeddings itself, from the caller's ids
    G2_TRY(encoder_launch(residual, next_ids_device, P(P_WTE), P(P_WPE) + (size_t)pos * cs, B, 1, C, V));
  const size_t plane = (size_t)m->kv_batch * c.max_seq_len * cs;
  if (persistent) {
    // one persistent kernel for the whole step
    DecodeStep st;
    st.wte = P(P_WTE);
    st.wpe_row = P(P_WPE) + (size_t)pos * cs;
    st.ln1w = P(P_LN1W);
    st.ln1b = P(P_LN1B);
    st.qkvw = P(P_QKVW);
    st.qkvb = P(P_QKVB);
    st.attprojw = P(P_ATTPROJW);
    st.attprojb = P(P_ATTPROJB);
    st.ln2w = P(P_LN2W);
    st.ln2b = P(P_LN2B);
    st.fcw = P(P_FCW);
    st.fcb = P(P_FCB);
    st.fcprojw = P(P_FCPROJW);
    st.fcprojb = P(P_FCPROJB);
    st.lnfw = P(P_LNFW);
    st.lnfb = P(P_LNFB);
    st.ids = next_ids_device;  // read in stream order, like a copy of them would be
    st.kv = m->kv;
    st.plane = plane;
    st.x = m->step_act;
    st.qkv = m->qkv;
    st.atty = m->step_act + (size_t)kDecodeMaxBatch * cs;
    st.h = m->step_act + (size_t)kDecodeMaxBatch * 2 * cs;
    st.att_part = m->step_act + (size_t)kDecodeMaxBatch * 6 * cs;
    st.att_ml = st.att_part + (size_t)kDecodeMaxBatch * kDecodeMaxSplits * cs;
    st.att_splits = decode_step_attention_splits(c, B, pos);
    st.logits = m->step_logits;
    st.flags = m->step_flags;
    st.epoch0 = m->step_epoch;
    st.spin_limit = m->step_spin_limit;
    st.trace = trace;
    st.B = B;
    st.C = C;
    st.L = L;
    st.NH = NH;
    st.V = V;
    st.pos = pos;
    st.maxT = c.max_seq_len;
    st.error_host = m->step_error_device;
    G2_TRY(decode_step_launch(st, c, m->device));
    m->step_epoch += 5u * (unsigned)L + 8u;
    // (no copy of the error word: the workgroup that gives up writes it to the pinned host word itself)
    m->step_stream = stream();
    m->step_pending = true;
  } else if (skinny_supported(B, C, true, residual, m->params) && skinny_supported(B, 4 * C, false, m->fch, m->params)) {
    // Up to 16 sequences: five launches per block.  The layernorms run inside the GEMMs
    // that consume them and the residual adds inside the GEMMs that produce the update:
    //   qkv = LN1(x) Wqkv ; attention ; x += atty Wproj ; h = gelu(LN2(x) Wfc) ; x += h Wfcproj
    float* x = residual;
    for (int l = 0; l < L; l++) {
      G2_TRY(skinny_launch(m->qkv, x, P(P_QKVW) + l * 3 * cs * cs, P(P_QKVB) + l * 3 * cs,
                           P(P_LN1W) + l * cs, P(P_LN1B) + l * cs, nullptr, B, C, 3 * C, false));
      G2_TRY(attention_decode_launch(m->atty, m->qkv, m->kv + (2 * (size_t)l) * plane,
                                     m->kv + (2 * (size_t)l + 1) * plane, B, pos, c.max_seq_len, C, NH));
      G2_TRY(skinny_launch(x, m->atty, P(P_ATTPROJW) + l * cs * cs, P(P_ATTPROJB) + l * cs, nullptr,
                           nullptr, x, B, C, C, false));
      G2_TRY(skinny_launch(m->fch, x, P(P_FCW) + l * 4 * cs * cs, P(P_FCB) + l * 4 * cs,
                           P(P_LN2W) + l * cs, P(P_LN2B) + l * cs, nullptr, B, C, 4 * C, true));
      G2_TRY(skinny_launch(x, m->fch, P(P_FCPROJW) + l * 4 * cs * cs, P(P_FCPROJB) + l * cs, nullptr,
                           nullptr, x, B, 4 * C, C, false));
    }
    G2_TRY(skinny_launch(m->step_logits, x, P(P_WTE), nullptr, P(P_LNFW), P(P_LNFB), nullptr, B, C, V,
                         false));
  } else {
    // More sequences (or sizes the fused kernel does not take): the launchers of the full pass
    // (beyond 16 sequences the GEMMs are tiled ones and may split K through the workspace).
    G2_TRY(begin_splitk_use(m));
    G2_TRY(layernorm_forward_status(m->ln, nullptr, nullptr, residual, P(P_LN1W), P(P_LN1B), B, 1, C));
    for (int l = 0; l < L; l++) {
      G2_TRY(matmul_forward_splitk_status(m->qkv, m->ln, P(P_QKVW) + l * 3 * cs * cs, P(P_QKVB) + l * 3 * cs,
                                          B, 1, C, 3 * C, 0, m->splitk, m->splitk_bytes));
      G2_TRY(attention_decode_launch(m->atty, m->qkv, m->kv + (2 * (size_t)l) * plane,
                                     m->kv + (2 * (size_t)l + 1) * plane, B, pos, c.max_seq_len, C, NH));
      G2_TRY(matmul_forward_splitk_status(m->proj, m->atty, P(P_ATTPROJW) + l * cs * cs, P(P_ATTPROJB) + l * cs,
                                          B, 1, C, C, 0, m->splitk, m->splitk_bytes));
      G2_TRY(fused_residual_layernorm_forward_status(other, m->ln, nullptr, nullptr, residual, m->proj,
                                                     P(P_LN2W) + l * cs, P(P_LN2B) + l * cs, B, 1, C));
      G2_TRY(matmul_forward_splitk_status(m->fch, m->ln, P(P_FCW) + l * 4 * cs * cs, P(P_FCB) + l * 4 * cs,
                                          B, 1, C, 4 * C, 1, m->splitk, m->splitk_bytes));
      G2_TRY(matmul_forward_splitk_status(m->proj, m->fch, P(P_FCPROJW) + l * 4 * cs * cs,
                                          P(P_FCPROJB) + l * cs, B, 1, 4 * C, C, 0, m->splitk, m->splitk_bytes));
      const float* nw = (l + 1 < L) ? P(P_LN1W) + (l + 1) * cs : P(P_LNFW);
      const float* nb = (l + 1 < L) ? P(P_LN1B) + (l + 1) * cs : P(P_LNFB);
      G2_TRY(fused_residual_layernorm_forward_status(residual, m->ln, nullptr, nullptr, other, m->proj,
                                                     nw, nb, B, 1, C));
    }
    G2_TRY(matmul_forward_splitk_status(m->step_logits, m->ln, P(P_WTE), nullptr, B, 1, C, V, 0, m->splitk,
                                        m->splitk_bytes));
    m->splitk_dirty = false;
  }
#undef G2_TRY
  m->kv_len = pos + 1;
  m->last_has_logits = false;  // the (B,T,V) buffer and the activations no longer describe a full pass
  return GPT2HIP_OK;
}
}  // namespace g2

int gpt2_decode_options(GPT2* model, int persistent, unsigned spin_limit) {
  if (!model) return g2::fail(GPT2HIP_EINVAL, "gpt2_decode_options: null model");
  // A failed step nobody has asked about yet is settled first (cache rolled back, barrier state
  // cleared): settling it later would switch the persistent kernel off again behind this
  // call's back.  Its failure is still reported, by this call's return value.
  const int pending = g2::settle_steps(model, true);
  if (persistent != 0) model->step_fallback = false;  // asked for (again) explicitly
  model->step_persistent = persistent != 0;
  model->step_spin_limit = spin_limit;
  return pending;
}

const float* gpt2_step_logits(const GPT2* model) { return model ? model->step_logits : nullptr; }
int gpt2_cache_length(const GPT2* model) { return model ? model->kv_len : 0; }

int gpt2_forward_argmax_status(GPT2* model, const int* inputs_device, int B, int T,
                               int* next_ids_device) {
  using namespace g2;
  if (int rc = reserve(model, B, T)) return rc;
  if (!inputs_device || !next_ids_device)
    return fail(GPT2HIP_EINVAL, "gpt2_forward_argmax: null pointer");
  G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                        hipMemcpyDeviceToDevice, stream()));
  return forward_resident(model, B, T, nullptr, next_ids_device);
}

int gpt2_forward_profiled_status(GPT2* model, const int* inputs_device, int B, int T,
                                 float* ms_per_category) {
  using namespace g2;
  if (int rc = reserve(model, B, T)) return rc;
  if (!inputs_device || !ms_per_category)
    return fail(GPT2HIP_EINVAL, "gpt2_forward_profiled: null pointer");
  G2_HIP(hipMemcpyAsync(model->ids, inputs_device, (size_t)B * T * sizeof(int),
                        hipMemcpyDeviceToDevice, stream()));
  // The pass's first launch, issued a few times untimed (it is idempotent): the opening event
  // then sits between back-to-back launches like every other event of the pass, instead of
  // behind the copy of the ids and the device's wake-up from idle, and the device is still busy
  // with them while the host queues that event and the first timed launch.
  Profile prof;
  for (int i = 0; i < 4; i++)
    if (int rc = encoder_launch(model->res_a, model->ids, model->params + model->param_off[P_WTE],
                                model->params + model->param_off[P_WPE], B, T, model->cfg.channels,
                                model->cfg.vocab_size))
      return rc;
  if (int rc = forward_resident(model, B, T, &prof)) return rc;
  G2_HIP(hipEventSynchronize(prof.events[prof.used - 1]));
  for (int i = 0; i < GPT2_PROF_COUNT; i++) ms_per_category[i] = 0.f;
  for (size_t i = 0; i < prof.category.size(); i++) {
    float ms = 0.f;
    G2_HIP(hipEventElapsedTime(&ms, prof.events[i], prof.events[i + 1]));
    ms_per_category[prof.category[i]] += ms;
  }
  return GPT2HIP_OK;
}

float gpt2hip_profile_marker_overhead_us(int launches) {
  using namespace g2;
  if (launches < 1) launches = 64;
  float* buf = nullptr;
  if (hipMalloc((void**)&buf, 256 * sizeof(float)) != hipSuccess) {
    fail(GPT2HIP_ENOMEM, "gpt2hip_profile_marker_overhead_us: hipMalloc failed");
    return -1.f;
  }
  float result = -1.f;
  do {
    if (hipMemsetAsync(buf, 0, 256 * sizeof(float), stream()) != hipSuccess) break;
    for (int i = 0; i < launches; i++)
      if (residual_forward_status(buf, buf, buf, 256)) break;
    // (a) an event after every launch, as gpt2_forward_profiled_status records them
    Profile prof;
    if (prof.mark(-1)) break;
    bool ok = true;
    for (int i = 0; i < launches && ok; i++) ok = !residual_forward_status(buf, buf, buf, 256) && !prof.mark(0);
    if (!ok || hipEventSynchronize(prof.events[prof.used - 1]) != hipSuccess) break;
    float marked = 0.f;
    if (hipEventElapsedTime(&marked, prof.events.front(), prof.events[prof.used - 1]) != hipSuccess) break;
    // (b) the same launches back to back between two events
    Profile bare;
    if (bare.mark(-1)) break;
    for (int i = 0; i < launches && ok; i++) ok = !residual_forward_status(buf, buf, buf, 256);
    if (!ok || bare.mark(0) || hipEventSynchronize(bare.events[bare.used - 1]) != hipSuccess) break;
    float plain = 0.f;
    if (hipEventElapsedTime(&plain, bare.events.front(), bare.events[bare.used - 1]) != hipSuccess) break;
    result = (marked - plain) * 1000.f / (float)launches;
    if (result < 0.f) result = 0.f;
  } while (false);
  (void)hipFree(buf);
  if (result < 0.f) fail(GPT2HIP_EHIP, "gpt2hip_profile_marker_overhead_us: a HIP call failed");
  return result;
}

const float* gpt2_logits(const GPT2* model) { return model ? model->logits : nullptr; }
const float* gpt2_lnf(const GPT2* model) { return model ? model->ln : nullptr; }

int gpt2_argmax_status(GPT2* model, int* ids_device) {
  using namespace g2;
  if (!model || !model->logits || model->last_B == 0 || !model->last_has_logits)
    return fail(GPT2HIP_EINVAL, "gpt2_argmax: no forward pass has left logits");
  return argmax_forward_status(ids_device, model->logits, model->last_B * model->last_T,
                               model->cfg.vocab_size);
}

// ---- event timer on the null stream ---------------------------------------
struct GPT2Timer {
  hipEvent_t start, stop;
};

GPT2Timer* gpt2hip_timer_create(void) {
  GPT2Timer* t = new GPT2Timer();
  if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) {
    g2::fail(GPT2HIP_EHIP, "gpt2hip_timer_create: hipEventCreate failed");
    delete t;
    return nullptr;
  }
  return t;
}

void gpt2hip_timer_destroy(GPT2Timer* t) {
  if (!t) return;
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
}

int gpt2hip_timer_start(GPT2Timer* t) {
  if (!t) return g2::fail(GPT2HIP_EINVAL, "gpt2hip_timer_start: null timer");
  G2_HIP(hipEventRecord(t->start, g2::stream()));
  return GPT2HIP_OK;
}

float gpt2hip_timer_stop_ms(GPT2Timer* t) {
  if (!t) return -1.f;
  float ms = -1.f;
  if (hipEventRecord(t->stop, g2::stream()) != hipSuccess || hipEventSynchronize(t->stop) != hipSuccess ||
      hipEventElapsedTime(&ms, t->start, t->stop) != hipSuccess) {
    g2::fail(GPT2HIP_EHIP, "gpt2hip_timer_stop_ms: event timing failed");
    return -1.f;
  }
  return ms;
}

}  // extern "C"
