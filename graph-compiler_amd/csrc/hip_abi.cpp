// The thin C-ABI layer between host code and the HIP kernels: argument
// validation, parameter-block assembly, launches.  This and the kernels' own
// launch stubs are the only translation units that touch the HIP runtime for
// compute.  Device memory is allocated in one place only: the library workspace of the entry points that take no
// workspace argument (LibraryWorkspace below).
#include <hip/hip_runtime_api.h>

#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <shared_mutex>
#include <vector>

#include "gc_brgemm.h"
#include "gc_hip_kernels.h"
#include "kernels/gemm_params.h"

using namespace gcmi;

extern "C" {
int gcmi_launch_gemm_bf16(const GemmParams *p, hipStream_t stream);
int gcmi_launch_gemm_int8(const GemmParams *p, hipStream_t stream);
int gcmi_launch_colsum_s8(const void *W, int64_t K, int64_t N, int64_t ldw, void *out, hipStream_t stream);
int gcmi_launch_gemm_f32(const F32GemmParams *p, hipStream_t stream);
int gcmi_launch_brgemm(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t LDA,
                       int64_t LDB, int64_t LDC, int64_t stride_a, int64_t stride_b, int num, int beta_zero, int dtA,
                       int dtB, hipStream_t stream);
int gcmi_launch_mha_fwd(const MhaParams *p, hipStream_t stream);
int64_t gcmi_launch_gemm_bf16_workspace(const GemmParams *p);
int gcmi_launch_gemm_bf16_config(const GemmParams *p, GemmTileConfig *cfg);
int gcmi_launch_gemm_int8_config(const GemmParams *p, GemmTileConfig *cfg);
int64_t gcmi_launch_mha_workspace(const MhaParams *p);
int gcmi_noalloc_scratch(void **ptr, size_t *bytes);
}

namespace {
thread_local char g_err[256] = "";
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
enum { ST_OK = 0, ST_INVALID = 2, ST_UNIMPL = 3, ST_RUNTIME = 5 };
int launched(int rc, const char *what) {
  if (rc == 0)
    return ST_OK;
  return fail(rc, "%s: launch failed (%s)", what, hipGetErrorString(hipPeekAtLastError()));
}
} // namespace

extern "C" const char *gcmi_last_error(void) { return g_err; }

namespace {
// Where a call's scratch (partial sums of K-sliced GEMMs, mask tile classes of attention) comes from.
enum class Ws { Library, Caller, Static };

// Scratch of the entry points that take no workspace argument: one buffer per device, allocated at the first call
// that needs it and grown on demand.  Every call on the device shares it, so its users are put in order: the mutex
// is held while a call's kernels are enqueued, an event is recorded behind them, and a call on another stream
// waits for that event first.
struct LibraryWorkspace {
  std::mutex mu;
  void *ptr = nullptr;
  size_t cap = 0;
  hipEvent_t done = nullptr;
  hipStream_t last = nullptr;
  bool used = false;
  // Blocks that were outgrown.  They are kept until the process ends: a kernel enqueued earlier (or a HIP graph
  // captured from an earlier call through an entry point that did not refuse capture) may still name them.
  std::vector<void *> retired;
};
LibraryWorkspace g_ws[64];

// hipStreamPerThread is one handle value for a different stream in every thread, and the legacy null stream
// synchronises with others by rules of its own: a comparison of handles says nothing about them.
bool same_stream_for_sure(hipStream_t a, hipStream_t b) {
  return a == b && a != nullptr && a != hipStreamPerThread && a != hipStreamLegacy;
}

// Takes the device's buffer (at least `bytes`) for one call on `stream`; the lock is held until release().
int ws_acquire(size_t bytes, hipStream_t stream, LibraryWorkspace **out, void **ptr) {
  // Under stream capture nothing here is legal (allocation, device-wide waits), and a captured graph would keep the
  // address of a buffer that later calls share: such callers bring their own workspace.
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
    (void)hipGetLastError();
    cap = hipStreamCaptureStatusNone;
  }
  if (cap != hipStreamCaptureStatusNone)
    return fail(ST_INVALID, "this call needs scratch memory and its stream is being captured: use the entry point that takes "
                            "a workspace (gcmi_gemm_bf16_ws / gcmi_mha_fwd_bf16_ws) or gcmi_gemm_bf16_noalloc");
  // the buffer of the device the stream belongs to (the current device for the null and per-thread streams)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return fail(ST_RUNTIME, "workspace: no current device");
  if (stream != nullptr && stream != hipStreamPerThread && stream != hipStreamLegacy) {
    hipDevice_t sdev = 0;
    if (hipStreamGetDevice(stream, &sdev) == hipSuccess && (int)sdev >= 0 && (int)sdev < 64)
      dev = (int)sdev;
    else
      (void)hipGetLastError();
  }
  LibraryWorkspace &w = g_ws[dev];
  w.mu.lock();
  if (w.cap < bytes) {
    const size_t want = bytes < ((size_t)8 << 20) ? ((size_t)8 << 20) : bytes;
    void *fresh = nullptr;
    if (hipMalloc(&fresh, want) != hipSuccess) {
      w.mu.unlock();
      return fail(1, "workspace: hipMalloc of %zu bytes failed", want);
    }
    if (w.ptr)
      w.retired.push_back(w.ptr); // never freed: see above
    w.ptr = fresh, w.cap = want;
    // the new block has no earlier user, but the order between callers is kept as it was (w.used, w.last)
  }
  if (!w.done && hipEventCreateWithFlags(&w.done, hipEventDisableTiming) != hipSuccess) {
    w.done = nullptr;
    w.mu.unlock();
    return fail(ST_RUNTIME, "workspace: hipEventCreate failed");
  }
  // A caller on another stream than the last user's waits for everything that stream has been given so far (the
  // marker is recorded now, behind the last user's kernels: nothing is recorded per call, so a single-stream caller
  // pays for no event).  A stream that no longer exists: wait for the device.
  if (w.used && !same_stream_for_sure(w.last, stream)) {
    if (hipEventRecord(w.done, w.last) != hipSuccess || hipStreamWaitEvent(stream, w.done, 0) != hipSuccess) {
      (void)hipGetLastError();
      (void)hipDeviceSynchronize();
    }
  }
  *out = &w, *ptr = w.ptr;
  return ST_OK;
}
void ws_release(LibraryWorkspace *w, hipStream_t stream) {
  w->used = true, w->last = stream;
  w->mu.unlock();
}
} // namespace

extern "C" int gcmi_init(int device) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0)
    return fail(ST_RUNTIME, "no HIP device visible");
  if (device < 0 || device >= n)
    return fail(ST_INVALID, "device %d out of range (%d visible)", device, n);
  if (hipSetDevice(device) != hipSuccess)
    return fail(ST_RUNTIME, "hipSetDevice(%d) failed", device);
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess)
    return fail(ST_RUNTIME, "hipGetDeviceProperties failed");
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(ST_UNIMPL, "device is %s; these kernels are built for gfx950 only", prop.gcnArchName);
  // the device address of the static scratch array (gcmi_gemm_bf16_noalloc), once per device
  void *sp = nullptr;
  size_t sb = 0;
  if (gcmi_noalloc_scratch(&sp, &sb) != 0)
    return fail(ST_RUNTIME, "hipGetSymbolAddress(scratch) failed on device %d", device);
  return ST_OK;
}

namespace {
// The reference reads a MatmulConfig from nine integer attributes of the matmul op -- all nine or none
// (readConfigFromAttrs, lib/gc/Analysis/MatmulConfigAnalysis.cpp:368-404) -- and drops it when validateConfig
// (:40-65) fails.  Here the nine are {MThreads, NThreads, KThreads, MBlock, NBlock, KBlock, innermostMBlock,
// innermostNBlock, innermostKBlock}; what they can steer on the GPU: the workgroup tile (MBlock x NBlock: 256 x 256
// is the one that is built), the tile of one wave (innermostMBlock x innermostNBlock: 128 x 128 = 4 waves per
// workgroup, 128 x 64 = 8 waves) and the number of K slices (KThreads).  MThreads x NThreads is the reference's
// thread grid; the GPU's grid follows from the tile.  Returns false, with the reason, when the config is not used.
bool apply_matmul_config(const int64_t *c, int64_t M, int64_t N, int64_t K, GemmParams &p, const char **why) {
  const int64_t MThreads = c[0], NThreads = c[1], KThreads = c[2], MBlock = c[3], NBlock = c[4], KBlock = c[5], iM = c[6],
                iN = c[7], iK = c[8];
  *why = "";
  for (int i = 0; i < 9; i++)
    if (c[i] <= 0) {
      *why = "invalid (a field is not positive)";
      return false;
    }
  (void)MThreads, (void)NThreads;
  if (MBlock % iM != 0 || NBlock % iN != 0 || KBlock % iK != 0) {
    *why = "invalid (a block is not a multiple of its innermost block)";
    return false;
  }
  if ((K + KBlock - 1) / KBlock < KThreads) {
    *why = "invalid (fewer K blocks than KThreads)";
    return false;
  }
  if (MBlock == 128 && NBlock == 128) { // the small tile: 4 waves of 64 x 64, no K slices
    if (iM != 64 || iN != 64) {
      *why = "not built (a wave's tile of the 128 x 128 workgroup tile is 64 x 64)";
      return false;
    }
    if (KThreads != 1) {
      *why = "not built (the 128 x 128 workgroup tile takes no K slices)";
      return false;
    }
    p.cfg_tile = 128;
    return true;
  }
  if (MBlock != 256 || NBlock != 256) {
    *why = "not built (the workgroup tile is 256 x 256 or 128 x 128)";
    return false;
  }
  if (iM != 128 || (iN != 128 && iN != 64)) {
    *why = "not built (a wave's tile is 128 x 128 or 128 x 64)";
    return false;
  }
  (void)M, (void)N;
  p.cfg_tile = 256;
  p.cfg_waves = iN == 128 ? 4 : 8;
  p.cfg_split_k = (int32_t)(KThreads > 1024 ? 1024 : KThreads);
  return true;
}

int gemm_bf16_any(bool trans_b, const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldb, int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype, void *stream,
                  int64_t batch = 1, int64_t a_bs = 0, int64_t b_bs = 0, int64_t c_bs = 0, const void *residual = nullptr,
                  int64_t ldr = 0, int residual_dtype = 0, Ws ws_from = Ws::Library, void *ws = nullptr,
                  size_t ws_bytes = 0, const int64_t *matmul_config = nullptr);
}

extern "C" int gcmi_gemm_bf16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                              int64_t ldb, int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype,
                              void *stream) {
  return gemm_bf16_any(false, A, B, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream);
}

extern "C" int gcmi_gemm_bf16_nt(const void *A, const void *Bt, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                                 int64_t ldb, int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype,
                                 void *stream) {
  return gemm_bf16_any(true, A, Bt, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream);
}

extern "C" int gcmi_gemm_bf16_batched(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N,
                                      int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
                                      int64_t stride_b, int64_t stride_c, int trans_b, const void *bias,
                                      int bias_dtype, int act, int out_dtype, void *stream) {
  if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
    return fail(ST_INVALID, "gemm_bf16_batched: negative batch count or stride");
  if (batch == 0)
    return ST_OK;
  if (batch > 65535)
    return fail(ST_UNIMPL, "gemm_bf16_batched: more than 65535 batches in one call");
  if (batch > 1 && stride_c < (M - 1) * ldc + N)
    return fail(ST_INVALID, "gemm_bf16_batched: results of different batches would overlap");
  return gemm_bf16_any(trans_b != 0, A, B, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream, batch,
                       stride_a, stride_b, stride_c);
}

extern "C" int gcmi_gemm_bf16_residual(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N,
                                       int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
                                       int64_t stride_b, int64_t stride_c, int trans_b, const void *bias,
                                       int bias_dtype, int act, const void *residual, int64_t ldr, int residual_dtype,
                                       int out_dtype, void *stream) {
  if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
    return fail(ST_INVALID, "gemm_bf16_residual: negative batch count or stride");
  if (batch == 0)
    return ST_OK;
  if (batch > 65535)
    return fail(ST_UNIMPL, "gemm_bf16_residual: more than 65535 batches in one call");
  if (batch > 1 && stride_c < (M - 1) * ldc + N)
    return fail(ST_INVALID, "gemm_bf16_residual: results of different batches would overlap");
  if (residual) {
    if (residual_dtype != GCMI_BF16 && residual_dtype != GCMI_F32)
      return fail(ST_UNIMPL, "gemm_bf16_residual: residual_dtype %d", residual_dtype);
    if (ldr < N || (batch > 1 && stride_c < (M - 1) * ldr + N))
      return fail(ST_INVALID, "gemm_bf16_residual: residual rows or batches overlap (ldr %lld)", (long long)ldr);
  }
  return gemm_bf16_any(trans_b != 0, A, B, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream, batch,
                       stride_a, stride_b, stride_c, residual, ldr, residual_dtype);
}

namespace {
int gemm_bf16_any(bool trans_b, const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldb, int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype, void *stream,
                  int64_t batch, int64_t a_bs, int64_t b_bs, int64_t c_bs, const void *residual, int64_t ldr,
                  int residual_dtype, Ws ws_from, void *ws, size_t ws_bytes, const int64_t *matmul_config) {
  if (M < 0 || N < 0 || K < 0)
    return fail(ST_INVALID, "gemm_bf16: negative size");
  if (M == 0 || N == 0)
    return ST_OK;
  if (!A || !B || !C)
    return fail(ST_INVALID, "gemm_bf16: null operand");
  if (lda < K || ldb < (trans_b ? K : N) || ldc < N)
    return fail(ST_INVALID, "gemm_bf16: leading dimension smaller than the row (lda %lld ldb %lld ldc %lld)",
                (long long)lda, (long long)ldb, (long long)ldc);
  if (out_dtype != GCMI_BF16 && out_dtype != GCMI_F32)
    return fail(ST_UNIMPL, "gemm_bf16: out_dtype %d", out_dtype);
  if (bias && bias_dtype != GCMI_BF16 && bias_dtype != GCMI_F32)
    return fail(ST_UNIMPL, "gemm_bf16: bias_dtype %d", bias_dtype);
  if (act < GCMI_ACT_NONE || act > GCMI_ACT_SIGMOID)
    return fail(ST_INVALID, "gemm_bf16: act %d", act);
  GemmParams p{};
  p.A = A, p.B = B, p.C = C, p.M = M, p.N = N, p.K = K, p.lda = lda, p.ldb = ldb, p.ldc = ldc;
  p.bias = bias, p.bias_dt = bias_dtype, p.act = act, p.out_dt = out_dtype;
  p.trans_b = trans_b ? 1 : 0;
  p.batch = batch, p.a_bs = a_bs, p.b_bs = b_bs, p.c_bs = c_bs;
  p.residual = residual, p.ldr = ldr, p.residual_dt = residual_dtype;
  if (matmul_config) {
    const char *why;
    (void)apply_matmul_config(matmul_config, M, N, K, p, &why); // not usable: ignored, as in the reference
  }
  // K-sliced shapes (a short A against wide weights) pass f32 partial sums through a workspace
  const int64_t want = gcmi_launch_gemm_bf16_workspace(&p);
  if (want <= 0)
    return launched(gcmi_launch_gemm_bf16(&p, (hipStream_t)stream), "gemm_bf16");
  if (ws_from == Ws::Caller) { // what the caller brought, however little: the launcher cuts fewer slices, or none
    if (ws && (reinterpret_cast<uintptr_t>(ws) & 15) != 0)
      return fail(ST_INVALID, "gemm_bf16: workspace is not 16-byte aligned");
    p.partial = ws_bytes >= 4 ? (float *)ws : nullptr, p.partial_cap = (int64_t)(ws_bytes / 4);
    return launched(gcmi_launch_gemm_bf16(&p, (hipStream_t)stream), "gemm_bf16");
  }
  if (ws_from == Ws::Static) {
    // the static array is per device and its address is the current device's: a stream of another device would be
    // handed the wrong GPU's address
    if (stream != nullptr && (hipStream_t)stream != hipStreamPerThread && (hipStream_t)stream != hipStreamLegacy) {
      int cur = -1;
      hipDevice_t sdev = -1;
      if (hipGetDevice(&cur) == hipSuccess && hipStreamGetDevice((hipStream_t)stream, &sdev) == hipSuccess && (int)sdev != cur)
        return fail(ST_INVALID, "gemm_bf16_noalloc: the stream belongs to device %d, the current device is %d; make the "
                                "stream's device current (hipSetDevice) before the call", (int)sdev, cur);
      (void)hipGetLastError();
    }
    void *sp = nullptr;
    size_t sb = 0;
    if (gcmi_noalloc_scratch(&sp, &sb) != 0)
      return fail(ST_RUNTIME, "gemm_bf16_noalloc: the address of the static scratch array is not available");
    if ((size_t)want * 4 > sb)
      return fail(ST_INVALID,
                  "gemm_bf16_noalloc: %lld x %lld x %lld needs %lld bytes of scratch for its K slices, the static "
                  "buffer holds %zu; use gcmi_gemm_bf16 (library workspace) or gcmi_gemm_bf16_ws",
                  (long long)M, (long long)N, (long long)K, (long long)want * 4, sb);
    p.partial = (float *)sp, p.partial_cap = (int64_t)(sb / 4);
    return launched(gcmi_launch_gemm_bf16(&p, (hipStream_t)stream), "gemm_bf16_noalloc");
  }
  LibraryWorkspace *lw = nullptr;
  void *lp = nullptr;
  if (int rc = ws_acquire((size_t)want * 4, (hipStream_t)stream, &lw, &lp))
    return rc;
  p.partial = (float *)lp, p.partial_cap = want;
  const int rc = launched(gcmi_launch_gemm_bf16(&p, (hipStream_t)stream), "gemm_bf16");
  ws_release(lw, (hipStream_t)stream);
  return rc;
}
} // namespace

extern "C" size_t gcmi_gemm_bf16_workspace_bytes_cfg(int64_t M, int64_t N, int64_t K, int trans_b,
                                                     const int64_t *matmul_config) {
  if (M <= 0 || N <= 0 || K <= 0)
    return 0;
  GemmParams p{};
  // aligned stand-ins: the question is what the shape could use
  p.A = p.B = (const void *)(uintptr_t)256, p.C = (void *)(uintptr_t)256;
  p.M = M, p.N = N, p.K = K, p.lda = K, p.ldb = trans_b ? K : N, p.ldc = N;
  p.bias_dt = GCMI_BF16, p.out_dt = GCMI_BF16, p.trans_b = trans_b ? 1 : 0, p.batch = 1;
  if (matmul_config) { // the slices a caller's MatmulConfig names, exactly as gcmi_gemm_bf16_ws will apply it
    const char *why;
    (void)apply_matmul_config(matmul_config, M, N, K, p, &why);
  }
  const int64_t want = gcmi_launch_gemm_bf16_workspace(&p);
  return want > 0 ? (size_t)want * 4 : 0;
}

extern "C" size_t gcmi_gemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_b) {
  return gcmi_gemm_bf16_workspace_bytes_cfg(M, N, K, trans_b, nullptr);
}

extern "C" int gcmi_gemm_bf16_ws(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                                 int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b,
                                 int64_t stride_c, int trans_b, const void *bias, int bias_dtype, int act,
                                 const void *residual, int64_t ldr, int residual_dtype, int out_dtype, void *workspace,
                                 size_t workspace_bytes, const int64_t *matmul_config, void *stream) {
  if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
    return fail(ST_INVALID, "gemm_bf16_ws: negative batch count or stride");
  if (batch == 0)
    return ST_OK;
  if (batch > 65535)
    return fail(ST_UNIMPL, "gemm_bf16_ws: more than 65535 batches in one call");
  if (batch > 1 && stride_c < (M - 1) * ldc + N)
    return fail(ST_INVALID, "gemm_bf16_ws: results of different batches would overlap");
  if (residual) {
    if (residual_dtype != GCMI_BF16 && residual_dtype != GCMI_F32)
      return fail(ST_UNIMPL, "gemm_bf16_ws: residual_dtype %d", residual_dtype);
    if (ldr < N || (batch > 1 && stride_c < (M - 1) * ldr + N))
      return fail(ST_INVALID, "gemm_bf16_ws: residual rows or batches overlap (ldr %lld)", (long long)ldr);
  }
  return gemm_bf16_any(trans_b != 0, A, B, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream, batch,
                       stride_a, stride_b, stride_c, residual, ldr, residual_dtype, Ws::Caller, workspace,
                       workspace_bytes, matmul_config);
}

extern "C" int gcmi_gemm_tile_config_query(int a_dtype, int64_t M, int64_t N, int64_t K, int trans_b, int out_dtype,
                                           const int64_t *matmul_config, gcmi_gemm_tile_config *out, char *note,
                                           size_t note_len) {
  if (note && note_len)
    note[0] = 0;
  if (!out || M <= 0 || N <= 0 || K <= 0)
    return fail(ST_INVALID, "gemm_tile_config_query: bad arguments");
  const bool i8 = a_dtype == GCMI_S8 || a_dtype == GCMI_U8;
  if (!i8 && a_dtype != GCMI_BF16)
    return fail(ST_UNIMPL, "gemm_tile_config_query: a_dtype %d", a_dtype);
  GemmParams p{};
  // aligned stand-ins and every workspace the shape could use: the question is what the shape gets
  p.A = p.B = (const void *)(uintptr_t)256, p.C = (void *)(uintptr_t)256;
  p.M = M, p.N = N, p.K = K, p.lda = K, p.ldb = trans_b ? K : N, p.ldc = N;
  p.bias_dt = GCMI_BF16, p.out_dt = out_dtype, p.trans_b = trans_b ? 1 : 0, p.batch = 1;
  p.partial = (float *)(uintptr_t)256, p.partial_cap = INT64_MAX;
  if (matmul_config) {
    const char *why = "";
    if (!apply_matmul_config(matmul_config, M, N, K, p, &why) && note && note_len)
      snprintf(note, note_len, "MatmulConfig attributes ignored: %s", why);
  }
  GemmTileConfig c{};
  const int rc = i8 ? gcmi_launch_gemm_int8_config(&p, &c) : gcmi_launch_gemm_bf16_config(&p, &c);
  if (rc)
    return fail(rc, "gemm_tile_config_query: no kernel takes this call");
  static_assert(sizeof(gcmi_gemm_tile_config) == sizeof(GemmTileConfig), "the public struct mirrors GemmTileConfig");
  memcpy(out, &c, sizeof(c));
  return ST_OK;
}

extern "C" size_t gcmi_noalloc_scratch_bytes(void) {
  void *p = nullptr;
  size_t b = 0;
  return gcmi_noalloc_scratch(&p, &b) == 0 ? b : 0;
}

extern "C" int gcmi_gemm_bf16_noalloc(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K,
                                      int64_t lda, int64_t ldb, int64_t ldc, int trans_b, const void *bias,
                                      int bias_dtype, int act, int out_dtype, void *stream) {
  return gemm_bf16_any(trans_b != 0, A, B, C, M, N, K, lda, ldb, ldc, bias, bias_dtype, act, out_dtype, stream, 1, 0, 0,
                       0, nullptr, 0, 0, Ws::Static);
}

extern "C" int gcmi_gemm_int8(const void *A, int a_dtype, const void *W, void *C, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc, const int32_t *colsum, int32_t zp_a,
                              const float *scale, const float *bias, int act, int out_dtype, void *stream) {
  return gcmi_gemm_int8_cfg(A, a_dtype, W, C, M, N, K, lda, ldb, ldc, colsum, zp_a, scale, bias, act, out_dtype, nullptr,
                            stream);
}

extern "C" int gcmi_gemm_int8_cfg(const void *A, int a_dtype, const void *W, void *C, int64_t M, int64_t N, int64_t K,
                                  int64_t lda, int64_t ldb, int64_t ldc, const int32_t *colsum, int32_t zp_a,
                                  const float *scale, const float *bias, int act, int out_dtype,
                                  const int64_t *matmul_config, void *stream) {
  if (M < 0 || N < 0 || K < 0)
    return fail(ST_INVALID, "gemm_int8: negative size");
  if (M == 0 || N == 0)
    return ST_OK;
  if (!A || !W || !C)
    return fail(ST_INVALID, "gemm_int8: null operand");
  if (a_dtype != GCMI_U8 && a_dtype != GCMI_S8)
    return fail(ST_UNIMPL, "gemm_int8: a_dtype %d", a_dtype);
  if (lda < K || ldb < N || ldc < N)
    return fail(ST_INVALID, "gemm_int8: leading dimension smaller than the row");
  if (out_dtype != GCMI_S32 && out_dtype != GCMI_F32 && out_dtype != GCMI_BF16)
    return fail(ST_UNIMPL, "gemm_int8: out_dtype %d", out_dtype);
  if (act < GCMI_ACT_NONE || act > GCMI_ACT_SIGMOID)
    return fail(ST_INVALID, "gemm_int8: act %d", act);
  // The matrix cores multiply signed bytes.  u8 activations enter as
  // (a ^ 0x80) = a - 128, so acc_true = acc_mfma + 128*colsum, and the
  // zero-point compensation subtracts zp_a*colsum: both fold into one integer
  // factor of colsum.
  const int32_t shift = a_dtype == GCMI_U8 ? 128 : 0;
  const int32_t comp = out_dtype == GCMI_S32 ? shift : shift - zp_a;
  if (comp != 0 && !colsum)
    return fail(ST_INVALID, "gemm_int8: colsum is required for u8 activations or a non-zero zero point");
  GemmParams p{};
  p.A = A, p.B = W, p.C = C, p.M = M, p.N = N, p.K = K, p.lda = lda, p.ldb = ldb, p.ldc = ldc;
  p.bias = bias, p.bias_dt = GCMI_F32, p.scale = scale, p.colsum = comp ? colsum : nullptr, p.comp = comp;
  p.a_xor = a_dtype == GCMI_U8 ? 0x80808080u : 0u;
  p.act = out_dtype == GCMI_S32 ? GCMI_ACT_NONE : act, p.out_dt = out_dtype;
  if (matmul_config) {
    const char *why;
    (void)apply_matmul_config(matmul_config, M, N, K, p, &why); // not usable: ignored, as in the reference
  }
  return launched(gcmi_launch_gemm_int8(&p, (hipStream_t)stream), "gemm_int8");
}

extern "C" int gcmi_colsum_s8(const void *W, int64_t K, int64_t N, int64_t ldw, int32_t *colsum, void *stream) {
  if (K < 0 || N < 0 || ldw < N)
    return fail(ST_INVALID, "colsum_s8: bad shape");
  if (N == 0)
    return ST_OK;
  if (!W || !colsum)
    return fail(ST_INVALID, "colsum_s8: null operand");
  return launched(gcmi_launch_colsum_s8(W, K, N, ldw, colsum, (hipStream_t)stream), "colsum_s8");
}

extern "C" int gcmi_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                             int64_t ldb, int64_t ldc, int trans_a, int trans_b, const float *bias, int act,
                             void *stream) {
  return gcmi_gemm_f32_batched(A, B, C, 1, M, N, K, lda, ldb, ldc, 0, 0, 0, trans_a, trans_b, bias, act, stream);
}

extern "C" int gcmi_gemm_f32_batched(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N,
                                     int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a,
                                     int64_t stride_b, int64_t stride_c, int trans_a, int trans_b, const float *bias,
                                     int act, void *stream) {
  if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0)
    return fail(ST_INVALID, "gemm_f32: negative batch count or stride");
  if (batch == 0)
    return ST_OK;
  if (batch > 65535)
    return fail(ST_UNIMPL, "gemm_f32: more than 65535 batches in one call");
  if (batch > 1 && stride_c < (M - 1) * ldc + N)
    return fail(ST_INVALID, "gemm_f32: results of different batches would overlap");
  if (M < 0 || N < 0 || K < 0)
    return fail(ST_INVALID, "gemm_f32: negative size");
  if (M == 0 || N == 0)
    return ST_OK;
  if (!A || !B || !C)
    return fail(ST_INVALID, "gemm_f32: null operand");
  if (lda < (trans_a ? M : K) || ldb < (trans_b ? K : N) || ldc < N)
    return fail(ST_INVALID, "gemm_f32: leading dimension smaller than the row");
  if (act < GCMI_ACT_NONE || act > GCMI_ACT_SIGMOID)
    return fail(ST_INVALID, "gemm_f32: act %d", act);
  F32GemmParams p{};
  p.A = A, p.B = B, p.C = C, p.M = M, p.N = N, p.K = K;
  p.a_rs = trans_a ? 1 : lda, p.a_cs = trans_a ? lda : 1;
  p.b_rs = trans_b ? 1 : ldb, p.b_cs = trans_b ? ldb : 1;
  p.ldc = ldc, p.bias = bias, p.act = act, p.beta = 0.0f;
  p.batch = batch, p.a_bs = stride_a, p.b_bs = stride_b, p.c_bs = stride_c;
  return launched(gcmi_launch_gemm_f32(&p, (hipStream_t)stream), "gemm_f32");
}

extern "C" int gcmi_mha_fwd_bf16(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld,
                                 void *O, int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale, void *stream) {
  return gcmi_mha_fwd_bf16_opt(Q, K, V, mask, mask_ld, O, BH, Sq, Sk, D, scale, 1, stream);
}

namespace {
int mha_any(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld, void *O, int64_t BH,
            int64_t Sq, int64_t Sk, int64_t D, float scale, int skip_masked, void *stream, Ws ws_from, void *ws,
            size_t ws_bytes);
}

extern "C" int gcmi_mha_fwd_bf16_opt(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld,
                                     void *O, int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale,
                                     int skip_masked, void *stream) {
  return mha_any(Q, K, V, mask, mask_ld, O, BH, Sq, Sk, D, scale, skip_masked, stream, Ws::Library, nullptr, 0);
}

extern "C" int gcmi_mha_fwd_bf16_ws(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld,
                                    void *O, int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale, int skip_masked,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  return mha_any(Q, K, V, mask, mask_ld, O, BH, Sq, Sk, D, scale, skip_masked, stream, Ws::Caller, workspace,
                 workspace_bytes);
}

extern "C" int gcmi_mha_classify_mask(const float *mask, int64_t mask_ld, int64_t Sq, int64_t Sk, int64_t D, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  if (!mask || Sq <= 0 || Sk <= 0 || Sq > 0x7fffffff || Sk > 0x7fffffff)
    return fail(ST_INVALID, "mha_classify_mask: bad arguments");
  if (mask_ld < Sk)
    return fail(ST_INVALID, "mha_classify_mask: mask_ld < Sk");
  MhaParams p{};
  // aligned stand-ins for the operands the pass does not touch
  p.Q = p.K = p.V = (const void *)(uintptr_t)256, p.O = (void *)(uintptr_t)256;
  p.mask = mask, p.mask_ld = mask_ld, p.BH = 1, p.Sq = (int)Sq, p.Sk = (int)Sk, p.D = (int)D, p.scale = 1.0f;
  p.classes_mode = 2;
  const int64_t want = gcmi_launch_mha_workspace(&p);
  if (want <= 0)
    return ST_OK; // this shape has no mask classes: nothing to prepare
  if (!workspace || (int64_t)workspace_bytes < want)
    return fail(ST_INVALID, "mha_classify_mask: the workspace holds %zu bytes, %lld are needed (gcmi_mha_fwd_workspace_bytes)",
                workspace_bytes, (long long)want);
  p.tile_class = (uint8_t *)workspace, p.tile_class_cap = (int64_t)workspace_bytes;
  return launched(gcmi_launch_mha_fwd(&p, (hipStream_t)stream), "mha_classify_mask");
}

extern "C" size_t gcmi_mha_fwd_workspace_bytes(int64_t Sq, int64_t Sk, int64_t D, int has_mask) {
  if (!has_mask || Sq <= 0 || Sk <= 0 || Sq > 0x7fffffff || Sk > 0x7fffffff)
    return 0;
  MhaParams p{};
  p.mask = (const float *)(uintptr_t)256;
  p.Sq = (int)Sq, p.Sk = (int)Sk, p.D = (int)D;
  const int64_t want = gcmi_launch_mha_workspace(&p);
  return want > 0 ? (size_t)want : 0;
}

namespace {
int mha_any(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld, void *O, int64_t BH,
            int64_t Sq, int64_t Sk, int64_t D, float scale, int skip_masked, void *stream, Ws ws_from, void *ws,
            size_t ws_bytes) {
  if (BH < 0 || Sq < 0 || Sk < 0)
    return fail(ST_INVALID, "mha_fwd: negative size");
  if (D != 128 && D != 64)
    return fail(ST_UNIMPL, "mha_fwd: head_dim %lld (128 and 64 are built)", (long long)D);
  if (BH == 0 || Sq == 0)
    return ST_OK;
  if (Sk == 0)
    return fail(ST_INVALID, "mha_fwd: no keys");
  if (!Q || !K || !V || !O)
    return fail(ST_INVALID, "mha_fwd: null operand");
  if (mask && mask_ld < Sk)
    return fail(ST_INVALID, "mha_fwd: mask_ld < Sk");
  if (BH > 0x7fffffff || Sq > 0x7fffffff || Sk > 0x7fffffff)
    return fail(ST_INVALID, "mha_fwd: size too large");
  MhaParams p{};
  p.Q = Q, p.K = K, p.V = V, p.O = O, p.mask = mask, p.mask_ld = mask_ld;
  p.BH = (int)BH, p.Sq = (int)Sq, p.Sk = (int)Sk, p.D = (int)D, p.scale = scale;
  p.skip_masked = (skip_masked & 1) ? 1 : 0;
  // bit 1 (GCMI_MHA_CLASSES_VALID): the caller's workspace holds this mask's classes already
  p.classes_mode = (skip_masked & 2) ? 1 : 0;
  if ((skip_masked & 2) && (ws_from != Ws::Caller || !ws))
    return fail(ST_INVALID, "mha_fwd: GCMI_MHA_CLASSES_VALID needs the workspace that gcmi_mha_classify_mask filled");
  // the classes of the mask's tiles (constant 0, constant -inf, general) go through a small workspace
  const int64_t want = gcmi_launch_mha_workspace(&p);
  LibraryWorkspace *lw = nullptr;
  if (want > 0 && ws_from == Ws::Caller) {
    p.tile_class = (uint8_t *)ws, p.tile_class_cap = (int64_t)ws_bytes;
  } else if (want > 0) {
    void *lp = nullptr;
    if (int rc = ws_acquire((size_t)want, (hipStream_t)stream, &lw, &lp))
      return rc;
    p.tile_class = (uint8_t *)lp, p.tile_class_cap = want;
  }
  int rc = gcmi_launch_mha_fwd(&p, (hipStream_t)stream);
  if (lw)
    ws_release(lw, (hipStream_t)stream);
  if (rc == 2)
    return fail(ST_INVALID, "mha_fwd: Q/K/V/O must be 16-byte aligned");
  return launched(rc, "mha_fwd");
}
} // namespace

// ---------------------------------------------------------------------------
// Microkernel ABI: dispatch-once / execute-many, as the reference's runtime
// (lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmOnednn.cpp:74-168).
namespace {
struct BrgemmDesc {
  int64_t M, N, K, LDA, LDB, LDC, stride_a, stride_b;
  float beta;
  int64_t dtA, dtB;
};
std::shared_mutex g_brgemm_lock;
std::vector<BrgemmDesc> &brgemm_table() {
  static std::vector<BrgemmDesc> *t = new std::vector<BrgemmDesc>(); // never freed: handles stay valid at exit
  return *t;
}
bool brgemm_pair_ok(int64_t a, int64_t b) {
  auto i8 = [](int64_t d) { return d == GCMI_S8 || d == GCMI_U8; };
  return (a == GCMI_F32 && b == GCMI_F32) || (a == GCMI_BF16 && b == GCMI_BF16) || (i8(a) && i8(b));
}
} // namespace

extern "C" int64_t dnnl_brgemm_dispatch(int64_t M, int64_t N, int64_t K, int64_t LDA, int64_t LDB, int64_t LDC,
                                        int64_t stride_a, int64_t stride_b, float beta, int64_t dtypeA,
                                        int64_t dtypeB) {
  if (M < 0 || N < 0 || K < 0 || !brgemm_pair_ok(dtypeA, dtypeB)) {
    fail(ST_INVALID, "brgemm_dispatch: unsupported shape or dtype pair (%lld,%lld)", (long long)dtypeA,
         (long long)dtypeB);
    return -1;
  }
  std::unique_lock<std::shared_mutex> g(g_brgemm_lock);
  auto &t = brgemm_table();
  t.push_back(BrgemmDesc{M, N, K, LDA, LDB, LDC, stride_a, stride_b, beta, dtypeA, dtypeB});
  return (int64_t)t.size() - 1;
}

extern "C" void dnnl_brgemm_tileconfig(int64_t) {}
extern "C" void dnnl_brgemm_tilerelease(void) {}

extern "C" void dnnl_brgemm_execute(int64_t kernel, void *A, uint64_t A_offset, void *B, uint64_t B_offset, void *C,
                                    uint64_t C_offset, int num) {
  BrgemmDesc d;
  {
    std::shared_lock<std::shared_mutex> g(g_brgemm_lock);
    auto &t = brgemm_table();
    if (kernel < 0 || kernel >= (int64_t)t.size()) {
      fail(ST_INVALID, "brgemm_execute: invalid kernel handle %lld", (long long)kernel);
      return;
    }
    d = t[(size_t)kernel];
  }
  const int es = d.dtA == GCMI_F32 ? 4 : (d.dtA == GCMI_BF16 ? 2 : 1);
  const int ces = 4;
  const char *a = (const char *)A + A_offset * es;
  const char *b = (const char *)B + B_offset * es;
  char *c = (char *)C + C_offset * ces;
  int rc = gcmi_launch_brgemm(a, b, c, d.M, d.N, d.K, d.LDA, d.LDB, d.LDC, d.stride_a, d.stride_b, num,
                              d.beta == 0.0f ? 1 : 0, (int)d.dtA, (int)d.dtB, nullptr);
  if (rc)
    fail(rc, "brgemm_execute: launch failed");
}
