// C ABI of libesmoe.so: argument checks, schedule policy, kernel launches.
// Declarations and the reference entry points they replace: include/esmoe.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <unordered_map>
#include <vector>

#include "esmoe.h"
#include "gemm_args.h"
#include "schedule.h"

extern "C" int esmoe_launch_grouped_gemm(const esmoe::GemmArgs* args, int mx, int grid, hipStream_t stream);
extern "C" int esmoe_static_scratch(int32_t** ptr, size_t* bytes, int* max_experts);
extern "C" int esmoe_launch_mxfp8_quant(const void* in, int in_dtype, const int* problem_sizes,
                                        const int* expert_offsets, const int* blockscale_offsets, void* q, uint8_t* sf,
                                        int num_experts, long sf_rows, int k, int swiglu, long dense_rows,
                                        hipStream_t stream);

extern "C" int esmoe_launch_fp8_quant_act(const void* in, int in_dtype, void* q, float* scales, long total_rows, int k,
                                          hipStream_t stream);

extern "C" int esmoe_launch_fp8_quant_weight(const void* in, int in_dtype, void* q, float* scales, long rows, int k,
                                             hipStream_t stream);

extern "C" int esmoe_launch_route_metadata(const int* ids, long num_pairs, int first_expert, int num_experts, int n, int k,
                                           int* problem_sizes, int* expert_offsets, int* blockscale_offsets, int* dst_row,
                                           int* chunk_counts, hipStream_t stream);
extern "C" int esmoe_launch_permute_rows(const void* in, const int* dst_row, long num_pairs, int topk, long row_bytes,
                                         void* out, hipStream_t stream);

extern "C" int esmoe_launch_swiglu_quant(const void* in, int in_dtype, void* q, float* scales, long total_rows, int inter,
                                        hipStream_t stream);

namespace {

constexpr long kRouteChunk = 1024;   // pairs per wavefront in routing.hip

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

struct DeviceInfo {
  int valid = 0;
  int cus = 0;
  int is_gfx950 = 0;
};
DeviceInfo g_dev[64];
std::mutex g_dev_mu;

// Properties of the current device, queried once per device.
int current_device_info(DeviceInfo* out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice failed: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= 64) return fail(ESMOE_ERR_UNSUPPORTED_DEVICE, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_dev_mu);
  if (!g_dev[dev].valid) {
    hipDeviceProp_t prop;
    err = hipGetDeviceProperties(&prop, dev);
    if (err != hipSuccess) return fail((int)err, "hipGetDeviceProperties failed: %s", hipGetErrorString(err));
    g_dev[dev].cus = prop.multiProcessorCount;
    g_dev[dev].is_gfx950 = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    g_dev[dev].valid = 1;
  }
  *out = g_dev[dev];
  if (!out->is_gfx950) return fail(ESMOE_ERR_UNSUPPORTED_DEVICE, "libesmoe kernels are built for gfx950 only");
  return 0;
}

// ESMOE_* environment variables (tuning aids) are read once per process, on the first GEMM launch; a value the
// kernels cannot honour is reported by every launch instead of being applied.
struct Knobs {
  int big_mt_fp8 = 12, big_mt_mx = 12, order = 0, light_share = -1, narrow_tail = -1, self_schedule = 1;
  char error[160] = "";
};

const Knobs& knobs() {
  static const Knobs k = [] {
    Knobs r;
    auto env_int = [](const char* name, int dflt) {
      const char* v = getenv(name);
      return v && *v ? atoi(v) : dflt;
    };
    const char* big = getenv("ESMOE_BIG_MT");
    if (big && *big) {
      const int v = atoi(big);
      if (v == 8 || v == 12) r.big_mt_fp8 = r.big_mt_mx = v;
      else snprintf(r.error, sizeof(r.error), "ESMOE_BIG_MT=%s: full tiles are 8 or 12 x 16 rows", big);
    }
    r.order = env_int("ESMOE_ORDER", 0);
    if (r.order < 0 || r.order > 2) snprintf(r.error, sizeof(r.error), "ESMOE_ORDER must be 0, 1 or 2");
    r.light_share = env_int("ESMOE_LIGHT_SHARE", -1);
    if (r.light_share < -1 || r.light_share > 32) snprintf(r.error, sizeof(r.error), "ESMOE_LIGHT_SHARE must be in [-1, 32]");
    r.narrow_tail = env_int("ESMOE_NARROW_TAIL", -1);
    if (r.narrow_tail < -1 || r.narrow_tail > 65536) snprintf(r.error, sizeof(r.error), "ESMOE_NARROW_TAIL must be in [-1, 65536]");
    r.self_schedule = env_int("ESMOE_SELF_SCHEDULE", 1);
    if (r.self_schedule < 0 || r.self_schedule > 1) snprintf(r.error, sizeof(r.error), "ESMOE_SELF_SCHEDULE must be 0 or 1");
    return r;
  }();
  return k;
}

// Light items of a launch's tail that go out as two 128-column halves (schedule.h); about half a launch's workgroups.
constexpr int kNarrowTail = 128;

// Default schedule policy: the one the host mirrors describe.  kind: bit 0 mxfp8, bit 1 a fused SwiGLU epilogue.
esmoe::SchedPolicy default_policy(int force_bm, int kind) {
  const int mx = kind & 1;
  esmoe::SchedPolicy p;
  p.force_mt = force_bm / 16;
  // Full tiles are 192 rows for both kernels: the tallest tile whose ring (three weight stages, two token stages per
  // wavefront group) fits the 160 KB of LDS, which is what the hand-scheduled K block of the tall tiles needs.  (A
  // 256-row tile does more MFMA work per byte copied but only fits with two stages per operand and measured slower.)
  (void)mx;
  p.big_mt = 12;
  p.order = 0;
  p.light_share = -1;
  // the fused epilogues quantise blocks that need a whole 256-row tile, and a forced height has no light items
  p.narrow_tail = (force_bm == 0 && !(kind & 2)) ? kNarrowTail : 0;
  return p;
}

// Policy of a launch: the default with the environment's overrides.
esmoe::SchedPolicy launch_policy(int force_bm, int kind) {
  esmoe::SchedPolicy p = default_policy(force_bm, kind);
  const Knobs& k = knobs();
  p.big_mt = (kind & 1) ? k.big_mt_mx : k.big_mt_fp8;
  if (p.narrow_tail && k.narrow_tail >= 0) p.narrow_tail = k.narrow_tail;
  p.order = k.order;
  p.light_share = k.light_share;
  return p;
}

// Schedule workspaces owned by the library, one per (device, stream) that has called a GEMM entry point without a
// workspace.  They come out of chunks of kScratchSlots workspaces (room for ESMOE_MAX_EXPERTS experts each), zeroed
// when the chunk is allocated; every launch leaves the counters of its workspace zero again (the last workgroup out
// zeroes them), which is what lets those launches go without a schedule kernel.  A slot stays with its stream handle
// for the life of the process.  Only a chunk allocation calls hipMalloc: the first call on a device, and the first
// call of every kScratchSlots-th new stream after that.
constexpr int kScratchSlots = 16;
struct ScratchPool {
  std::mutex mu;
  std::unordered_map<hipStream_t, int32_t*> slot[64];   // by device
  std::vector<int32_t*> free_slots[64];
};
ScratchPool g_pool;

int library_scratch(hipStream_t stream, int32_t** ws, size_t* bytes) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice failed: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= 64) return fail(ESMOE_ERR_UNSUPPORTED_DEVICE, "device index %d out of range", dev);
  const size_t slot_bytes = esmoe_gemm_workspace_bytes(ESMOE_MAX_EXPERTS);
  std::lock_guard<std::mutex> lock(g_pool.mu);
  auto it = g_pool.slot[dev].find(stream);
  if (it == g_pool.slot[dev].end()) {
    if (g_pool.free_slots[dev].empty()) {
      void* chunk = nullptr;
      err = hipMalloc(&chunk, slot_bytes * kScratchSlots);
      if (err == hipSuccess) err = hipMemset(chunk, 0, slot_bytes * kScratchSlots);
      if (err != hipSuccess)
        return fail((int)err, "allocating the library's schedule workspaces failed: %s (the first call on a device, and of a "
                              "new stream once %d are in use, allocates: make it outside graph capture, or pass a workspace)",
                    hipGetErrorString(err), kScratchSlots);
      for (int i = kScratchSlots - 1; i >= 0; i--) g_pool.free_slots[dev].push_back((int32_t*)((char*)chunk + (size_t)i * slot_bytes));
    }
    it = g_pool.slot[dev].emplace(stream, g_pool.free_slots[dev].back()).first;
    g_pool.free_slots[dev].pop_back();
  }
  *ws = it->second;
  *bytes = slot_bytes;
  return 0;
}

int check_common(const void* out, const void* a, const void* b, const int32_t* ps, const int32_t* eo, int num_experts,
                 int total_rows, int n, int k, int force_bm, void* workspace, size_t workspace_bytes, int out_dtype) {
  if (!out || !a || !b || !ps || !eo) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if (num_experts < 1 || num_experts > ESMOE_MAX_EXPERTS)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "num_experts must be in [1, %d], got %d", ESMOE_MAX_EXPERTS, num_experts);
  if (n <= 0 || n % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "n must be a positive multiple of 128, got %d", n);
  if (k <= 0 || k % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must be a positive multiple of 128, got %d", k);
  if (k > 32768) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must be <= 32768, got %d", k);
  if (total_rows < 0) return fail(ESMOE_ERR_INVALID_ARGUMENT, "total_rows must be >= 0");
  if (out_dtype != ESMOE_OUT_BF16 && out_dtype != ESMOE_OUT_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "out_dtype must be ESMOE_OUT_BF16 or ESMOE_OUT_FP16");
  if (force_bm != 0 && force_bm != 16 && force_bm != 32 && force_bm != 64 && force_bm != 128 && force_bm != 192)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "force_bm must be 0, 16, 32, 64, 128 or 192, got %d", force_bm);
  // (workspace == NULL with workspace_bytes == 0: the library's own workspace of the stream, resolved at the launch)
  if (workspace || workspace_bytes) {
    if (!workspace || workspace_bytes < esmoe_gemm_workspace_bytes(num_experts))
      return fail(ESMOE_ERR_WORKSPACE_TOO_SMALL, "workspace of %zu bytes is smaller than the %zu required",
                  workspace_bytes, esmoe_gemm_workspace_bytes(num_experts));
    // (the kernel reads a schedule record with one 16-byte scalar load)
    if ((uintptr_t)workspace % 16) return fail(ESMOE_ERR_INVALID_ARGUMENT, "workspace must be 16-byte aligned");
  }
  if ((uintptr_t)a % 16 || (uintptr_t)b % 16 || (uintptr_t)out % 8)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "a and b must be 16-byte aligned, out 8-byte aligned");
  return 0;
}

// `owned`: g.ws is a workspace of the library (counters zero between launches), or null for the stream's own.
int launch_gemm(esmoe::GemmArgs& g, int mx, int force_bm, void* stream, bool owned = false) {
  if (g.total_rows == 0) return 0;
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  if (knobs().error[0]) return fail(ESMOE_ERR_INVALID_ARGUMENT, "%s", knobs().error);
  if (!g.ws) {
    size_t bytes = 0;
    rc = library_scratch((hipStream_t)stream, &g.ws, &bytes);
    if (rc) return rc;
    owned = true;
  }
  // One launch when the counters are known to be zero and a workgroup can rank the experts with a thread each.
  g.self_schedule = owned && knobs().self_schedule && g.num_experts <= esmoe::kSelfScheduleMaxExperts;
  g.policy = launch_policy(force_bm, (mx ? 1 : 0) | (g.q_out ? 2 : 0));
  // every height the schedule can hand out must be one the kernel has a tile function for (it has no other case)
  if ((g.policy.force_mt && !esmoe::sched_valid_mt(g.policy.force_mt)) || (g.policy.big_mt != 8 && g.policy.big_mt != 12))
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "tile heights %d / %d rows are not compiled into the kernels",
                g.policy.force_mt * 16, g.policy.big_mt * 16);
  int grid = info.cus;   // one persistent workgroup per CU: its LDS ring takes the whole 160 KB
  rc = esmoe_launch_grouped_gemm(&g, mx, grid, (hipStream_t)stream);
  if (rc) return fail(rc, "grouped GEMM launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

}  // namespace

extern "C" {

int esmoe_stream_workspace(void* stream, void** workspace, size_t* bytes) {
  g_err[0] = 0;
  if (!workspace || !bytes) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null pointer");
  int32_t* ws = nullptr;
  int rc = library_scratch((hipStream_t)stream, &ws, bytes);
  *workspace = ws;
  return rc;
}

size_t esmoe_gemm_workspace_bytes(int num_experts) {
  if (num_experts < 0) num_experts = 0;
  size_t bytes = (size_t)esmoe::ws_words(num_experts) * 4;
  return (bytes + 255) & ~(size_t)255;
}

int esmoe_fp8_blockwise_grouped_mm(void* out, int out_dtype, const void* a, const void* b, const float* sa,
                                   const float* sb, const int32_t* problem_sizes, const int32_t* expert_offsets,
                                   int num_experts, int total_rows, int n, int k, int force_bm, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = check_common(out, a, b, problem_sizes, expert_offsets, num_experts, total_rows, n, k, force_bm, workspace,
                        workspace_bytes, out_dtype);
  if (rc) return rc;
  if (!sa || !sb) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null scale pointer");
  esmoe::GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.sa = sa; g.sb = sb; g.out = out;
  g.problem_sizes = problem_sizes; g.expert_offsets = expert_offsets;
  g.ws = (int32_t*)workspace;
  g.num_experts = num_experts; g.total_rows = total_rows; g.n = n; g.k = k; g.out_dtype = out_dtype;
  return launch_gemm(g, 0, force_bm, stream);
}

int esmoe_fp8_blockwise_grouped_mm_static(void* out, int out_dtype, const void* a, const void* b, const float* sa,
                                          const float* sb, const int32_t* problem_sizes,
                                          const int32_t* expert_offsets, int num_experts, int total_rows, int n, int k,
                                          int force_bm, void* stream) {
  g_err[0] = 0;
  int32_t* ws = nullptr;
  size_t ws_bytes = 0;
  int max_experts = 0;
  int rc = esmoe_static_scratch(&ws, &ws_bytes, &max_experts);
  if (rc) return fail(rc, "static workspace lookup failed: %s", hipGetErrorString((hipError_t)rc));
  if (num_experts > max_experts)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "the static workspace holds the schedule of at most %d experts, got %d",
                max_experts, num_experts);
  rc = check_common(out, a, b, problem_sizes, expert_offsets, num_experts, total_rows, n, k, force_bm, ws, ws_bytes, out_dtype);
  if (rc) return rc;
  if (!sa || !sb) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null scale pointer");
  esmoe::GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.sa = sa; g.sb = sb; g.out = out;
  g.problem_sizes = problem_sizes; g.expert_offsets = expert_offsets;
  g.ws = ws;
  g.num_experts = num_experts; g.total_rows = total_rows; g.n = n; g.k = k; g.out_dtype = out_dtype;
  // the static array is zero when the library is loaded and every launch leaves its counters zero
  return launch_gemm(g, 0, force_bm, stream, /*owned=*/true);
}

int esmoe_fp8_blockwise_grouped_mm_swiglu_quant(void* q, float* scales, int mid_dtype, const void* a, const void* b,
                                                const float* sa, const float* sb, const int32_t* problem_sizes,
                                                const int32_t* expert_offsets, int num_experts, int total_rows, int n,
                                                int k, int force_bm, void* workspace, size_t workspace_bytes,
                                                void* stream) {
  g_err[0] = 0;
  int rc = check_common(q, a, b, problem_sizes, expert_offsets, num_experts, total_rows, n, k, force_bm, workspace,
                        workspace_bytes, mid_dtype);
  if (rc) return rc;
  if (!sa || !sb || !scales) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null scale pointer");
  if (n % 256) return fail(ESMOE_ERR_INVALID_ARGUMENT, "n = 2 * inter with inter a multiple of 128, got n = %d", n);
  if ((uintptr_t)q % 4 || (uintptr_t)scales % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "q and scales must be 4-byte aligned");
  esmoe::GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.sa = sa; g.sb = sb; g.q_out = q; g.scales_out = scales;
  g.problem_sizes = problem_sizes; g.expert_offsets = expert_offsets;
  g.ws = (int32_t*)workspace;
  g.num_experts = num_experts; g.total_rows = total_rows; g.n = n; g.k = k; g.out_dtype = mid_dtype;
  return launch_gemm(g, 0, force_bm, stream);
}

int esmoe_mxfp8_grouped_mm(void* d, int out_dtype, const void* a, const void* b, const uint8_t* sfa,
                           const uint8_t* sfb, const int32_t* problem_sizes, const int32_t* expert_offsets,
                           const int32_t* blockscale_offsets, int num_experts, int total_rows, int n, int k,
                           int force_bm, void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = check_common(d, a, b, problem_sizes, expert_offsets, num_experts, total_rows, n, k, force_bm, workspace,
                        workspace_bytes, out_dtype);
  if (rc) return rc;
  if (!sfa || !sfb || !blockscale_offsets) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null scale pointer");
  if ((uintptr_t)sfa % 4 || (uintptr_t)sfb % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "sfa and sfb must be 4-byte aligned");
  esmoe::GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.sfa = sfa; g.sfb = sfb; g.out = d;
  g.problem_sizes = problem_sizes; g.expert_offsets = expert_offsets; g.blockscale_offsets = blockscale_offsets;
  g.ws = (int32_t*)workspace;
  g.num_experts = num_experts; g.total_rows = total_rows; g.n = n; g.k = k; g.out_dtype = out_dtype;
  return launch_gemm(g, 1, force_bm, stream);
}

int esmoe_mxfp8_grouped_mm_swiglu_quant(void* q, uint8_t* sf, int mid_dtype, const void* a, const void* b,
                                        const uint8_t* sfa, const uint8_t* sfb, const int32_t* problem_sizes,
                                        const int32_t* expert_offsets, const int32_t* blockscale_offsets,
                                        int num_experts, int total_rows, int sf_rows, int n, int k, int force_bm,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = check_common(q, a, b, problem_sizes, expert_offsets, num_experts, total_rows, n, k, force_bm, workspace,
                        workspace_bytes, mid_dtype);
  if (rc) return rc;
  if (!sfa || !sfb || !sf || !blockscale_offsets) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null scale pointer");
  if ((uintptr_t)sfa % 4 || (uintptr_t)sfb % 4 || (uintptr_t)sf % 4 || (uintptr_t)q % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "sfa, sfb, sf and q must be 4-byte aligned");
  if (n % 256) return fail(ESMOE_ERR_INVALID_ARGUMENT, "n = 2 * inter with inter a multiple of 128, got n = %d", n);
  // every expert's scale rows are padded to 128, so sf holds at least the row total rounded up
  if (sf_rows % 128 || sf_rows < (total_rows + 127) / 128 * 128)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "sf_rows must be a multiple of 128 and >= total_rows rounded up to 128, got %d",
                sf_rows);
  esmoe::GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.b = b; g.sfa = sfa; g.sfb = sfb; g.q_out = q; g.sf_out = sf;
  g.problem_sizes = problem_sizes; g.expert_offsets = expert_offsets; g.blockscale_offsets = blockscale_offsets;
  g.ws = (int32_t*)workspace;
  g.num_experts = num_experts; g.total_rows = total_rows; g.n = n; g.k = k; g.out_dtype = mid_dtype;
  return launch_gemm(g, 1, force_bm, stream);
}

namespace {
int grouped_quant_common(const void* in, int in_dtype, const int32_t* problem_sizes, const int32_t* expert_offsets,
                         const int32_t* blockscale_offsets, void* q, uint8_t* sf, int num_experts, int total_rows,
                         int sf_rows, int k, int swiglu, void* stream) {
  g_err[0] = 0;
  if (!in || !problem_sizes || !expert_offsets || !blockscale_offsets || !q || !sf)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if (num_experts < 1 || num_experts > ESMOE_MAX_EXPERTS)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "num_experts must be in [1, %d], got %d", ESMOE_MAX_EXPERTS, num_experts);
  if (k <= 0 || k % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must align to 128, got %d", k);
  if (k > (1 << 20)) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must be <= 1048576, got %d", k);
  if (in_dtype != ESMOE_IN_BF16 && in_dtype != ESMOE_IN_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in_dtype must be ESMOE_IN_BF16 or ESMOE_IN_FP16");
  if (total_rows < 0 || sf_rows < 0 || sf_rows % 128)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "sf_rows must be a non-negative multiple of 128, got %d", sf_rows);
  if ((uintptr_t)in % 16 || (uintptr_t)q % 8 || (uintptr_t)sf % 16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in and sf must be 16-byte aligned, q 8-byte aligned");
  if (total_rows == 0 || sf_rows == 0) return 0;
  if (sf_rows / 128 > 65535)   // keeps the launch's workgroup count (32 rows x 256 columns each) far inside 2^31
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "sf_rows must not exceed 65535 * 128, got %d", sf_rows);
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_mxfp8_quant(in, in_dtype, problem_sizes, expert_offsets, blockscale_offsets, q, sf, num_experts,
                                sf_rows, k, swiglu, 0, (hipStream_t)stream);
  if (rc) return fail(rc, "quant launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}
}  // namespace

int esmoe_mxfp8_grouped_quant(const void* in, int in_dtype, const int32_t* problem_sizes,
                              const int32_t* expert_offsets, const int32_t* blockscale_offsets, void* q,
                              uint8_t* sf, int num_experts, int total_rows, int sf_rows, int k, void* stream) {
  return grouped_quant_common(in, in_dtype, problem_sizes, expert_offsets, blockscale_offsets, q, sf, num_experts,
                              total_rows, sf_rows, k, 0, stream);
}

int esmoe_swiglu_mxfp8_grouped_quant(const void* in, int in_dtype, const int32_t* problem_sizes,
                                     const int32_t* expert_offsets, const int32_t* blockscale_offsets, void* q,
                                     uint8_t* sf, int num_experts, int total_rows, int sf_rows, int inter,
                                     void* stream) {
  return grouped_quant_common(in, in_dtype, problem_sizes, expert_offsets, blockscale_offsets, q, sf, num_experts,
                              total_rows, sf_rows, inter, 1, stream);
}

int esmoe_mxfp8_quant_weight(const void* in, int in_dtype, void* q, uint8_t* sf, long rows, int k, void* stream) {
  g_err[0] = 0;
  if (k <= 0 || k % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must align to 128, got %d", k);
  if (k > (1 << 20)) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must be <= 1048576, got %d", k);
  if (in_dtype != ESMOE_IN_BF16 && in_dtype != ESMOE_IN_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in_dtype must be ESMOE_IN_BF16 or ESMOE_IN_FP16");
  if (rows < 0 || rows % 128 || rows / 128 > 65535)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "rows must be a non-negative multiple of 128, at most 65535 * 128, got %ld", rows);
  if (rows == 0) return 0;
  if (!in || !q || !sf) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if ((uintptr_t)in % 16 || (uintptr_t)q % 8 || (uintptr_t)sf % 16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in and sf must be 16-byte aligned, q 8-byte aligned");
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_mxfp8_quant(in, in_dtype, nullptr, nullptr, nullptr, q, sf, 1, rows, k, 0, rows, (hipStream_t)stream);
  if (rc) return fail(rc, "quant launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

int esmoe_fp8_quant_act_1x128(const void* in, int in_dtype, void* q, float* scales, long total_rows, int k, void* stream) {
  g_err[0] = 0;
  if (k <= 0 || k % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must align to 128, got %d", k);
  if (in_dtype != ESMOE_IN_BF16 && in_dtype != ESMOE_IN_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in_dtype must be ESMOE_IN_BF16 or ESMOE_IN_FP16");
  if (total_rows < 0 || total_rows > (1L << 40) / k)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "total_rows out of range: %ld", total_rows);
  if (total_rows == 0) return 0;   // empty tensors may carry null pointers
  if (!in || !q || !scales) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if ((uintptr_t)in % 16 || (uintptr_t)q % 8 || (uintptr_t)scales % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in must be 16-byte aligned, q 8-byte aligned, scales 4-byte aligned");
  if (total_rows == 0) return 0;
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_fp8_quant_act(in, in_dtype, q, scales, total_rows, k, (hipStream_t)stream);
  if (rc) return fail(rc, "quant launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

int esmoe_fp8_quant_weight_128x128(const void* in, int in_dtype, void* q, float* scales, long rows, int k, void* stream) {
  g_err[0] = 0;
  if (k <= 0 || k % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "k must align to 128, got %d", k);
  if (rows < 0 || rows % 128 || rows / 128 > 65535)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "rows must be a multiple of 128 in [0, 128 * 65535], got %ld", rows);
  if (in_dtype != ESMOE_IN_BF16 && in_dtype != ESMOE_IN_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in_dtype must be ESMOE_IN_BF16 or ESMOE_IN_FP16");
  if (rows == 0) return 0;
  if (!in || !q || !scales) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if ((uintptr_t)in % 16 || (uintptr_t)q % 8 || (uintptr_t)scales % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in must be 16-byte aligned, q 8-byte aligned, scales 4-byte aligned");
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_fp8_quant_weight(in, in_dtype, q, scales, rows, k, (hipStream_t)stream);
  if (rc) return fail(rc, "quant launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

int esmoe_swiglu_quant_1x128(const void* in, int in_dtype, void* q, float* scales, long total_rows, int inter,
                             void* stream) {
  g_err[0] = 0;
  if (inter <= 0 || inter % 128) return fail(ESMOE_ERR_INVALID_ARGUMENT, "inter must align to 128, got %d", inter);
  if (in_dtype != ESMOE_IN_BF16 && in_dtype != ESMOE_IN_FP16)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in_dtype must be ESMOE_IN_BF16 or ESMOE_IN_FP16");
  if (total_rows < 0 || total_rows > (1L << 40) / inter)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "total_rows out of range: %ld", total_rows);
  if (total_rows == 0) return 0;
  if (!in || !q || !scales) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if ((uintptr_t)in % 16 || (uintptr_t)q % 8 || (uintptr_t)scales % 4)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "in must be 16-byte aligned, q 8-byte aligned, scales 4-byte aligned");
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_swiglu_quant(in, in_dtype, q, scales, total_rows, inter, (hipStream_t)stream);
  if (rc) return fail(rc, "swiglu quant launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

size_t esmoe_route_workspace_bytes(long num_pairs, int num_experts) {
  if (num_pairs < 0) num_pairs = 0;
  if (num_experts < 1) num_experts = 1;
  const size_t chunks = (size_t)((num_pairs + kRouteChunk - 1) / kRouteChunk);
  const size_t bytes = (chunks ? chunks : 1) * (size_t)num_experts * 4;
  return (bytes + 255) & ~(size_t)255;
}

int esmoe_route_metadata(const int32_t* topk_ids, long num_pairs, int first_expert, int num_experts, int n, int k,
                         int32_t* problem_sizes, int32_t* expert_offsets, int32_t* blockscale_offsets,
                         int32_t* dst_row, void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  if (num_experts < 1 || num_experts > ESMOE_MAX_EXPERTS)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "num_experts must be in [1, %d], got %d", ESMOE_MAX_EXPERTS, num_experts);
  if (num_pairs < 0 || num_pairs >= (1L << 31))
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "num_pairs must be in [0, 2^31), got %ld", num_pairs);
  if (!problem_sizes || !expert_offsets || !blockscale_offsets || (num_pairs && (!topk_ids || !dst_row)))
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if (!workspace || workspace_bytes < esmoe_route_workspace_bytes(num_pairs, num_experts))
    return fail(ESMOE_ERR_WORKSPACE_TOO_SMALL, "workspace needs %zu bytes, got %zu",
                esmoe_route_workspace_bytes(num_pairs, num_experts), workspace_bytes);
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_route_metadata(topk_ids, num_pairs, first_expert, num_experts, n, k, problem_sizes, expert_offsets,
                                   blockscale_offsets, dst_row, (int*)workspace, (hipStream_t)stream);
  if (rc) return fail(rc, "routing launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

int esmoe_permute_rows(const void* in, const int32_t* dst_row, long num_pairs, int topk, long row_bytes, void* out,
                       void* stream) {
  g_err[0] = 0;
  if (num_pairs < 0 || topk < 1) return fail(ESMOE_ERR_INVALID_ARGUMENT, "num_pairs must be >= 0 and topk >= 1");
  if (row_bytes <= 0 || row_bytes % 16) return fail(ESMOE_ERR_INVALID_ARGUMENT, "row_bytes must be a positive multiple of 16");
  if (num_pairs == 0) return 0;
  if (!in || !dst_row || !out) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if ((uintptr_t)in % 16 || (uintptr_t)out % 16) return fail(ESMOE_ERR_INVALID_ARGUMENT, "in and out must be 16-byte aligned");
  DeviceInfo info;
  int rc = current_device_info(&info);
  if (rc) return rc;
  rc = esmoe_launch_permute_rows(in, dst_row, num_pairs, topk, row_bytes, out, (hipStream_t)stream);
  if (rc) return fail(rc, "permute launch failed: %s", hipGetErrorString((hipError_t)rc));
  return 0;
}

int esmoe_host_schedule(const int32_t* problem_sizes_host, int num_experts, int n, int force_bm, int kind,
                        int32_t* ws_host) {
  g_err[0] = 0;
  if (!problem_sizes_host || !ws_host || num_experts < 1 || num_experts > ESMOE_MAX_EXPERTS || n <= 0 || n % 128)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "bad argument to esmoe_host_schedule");
  const esmoe::SchedPolicy p = default_policy(force_bm, kind);
  auto rows_of = [&](int e) { return problem_sizes_host[e * 3] < 0 ? 0 : problem_sizes_host[e * 3]; };
  // same ranking as the device schedule kernel: by sched_order_key, ties by expert index
  for (int e = 0; e < num_experts; e++) {
    int pos = e;
    if (p.order != 1) {
      pos = 0;
      const int key = esmoe::sched_order_key(rows_of(e), p);
      for (int j = 0; j < num_experts; j++) {
        const int kj = esmoe::sched_order_key(rows_of(j), p);
        pos += (kj < key) || (kj == key && j < e);
      }
    }
    ws_host[esmoe::ws_rec(pos) + esmoe::kRecExpert] = e;
    ws_host[esmoe::ws_rec(pos) + esmoe::kRecRows] = rows_of(e);
  }
  int blocks = 0, items = 0;
  long heavy_cost = 0, light_cost = 0;
  for (int pos = 0; pos < num_experts; pos++) {
    const int m = ws_host[esmoe::ws_rec(pos) + esmoe::kRecRows];
    ws_host[esmoe::ws_rec(pos) + esmoe::kRecBlock] = blocks;
    ws_host[esmoe::ws_rec(pos) + esmoe::kRecItem] = items;
    blocks += esmoe::sched_heavy_blocks(m, n, p);
    items += esmoe::sched_light_items(m, n, p);
    heavy_cost += esmoe::sched_heavy_cost(m, n, p);
    light_cost += esmoe::sched_light_cost(m, n, p);
  }
  int32_t* last = ws_host + esmoe::ws_rec(num_experts);
  last[esmoe::kRecBlock] = blocks;
  last[esmoe::kRecItem] = items;
  last[esmoe::kRecExpert] = -1;
  last[esmoe::kRecRows] = 0;
  ws_host[esmoe::kWsLightShare] = esmoe::sched_light_share(heavy_cost, light_cost, p);
  ws_host[esmoe::kWsHeavyBlocks] = blocks;
  const int split = esmoe::sched_light_split(items, p);
  ws_host[esmoe::kWsLightSplit] = split;
  ws_host[esmoe::kWsLightTotal] = split + 2 * (items - split);
  ws_host[esmoe::kWsLightCounter] = 0;
  for (int x = 0; x < esmoe::kXcds; x++) ws_host[esmoe::ws_xcd_counter(x)] = 0;
  return 0;
}

namespace {
// Schedule position whose [first, next) range of blocks (kind kRecBlock) or items (kRecItem) holds v.
int host_position(const int32_t* ws_host, int num, int kind, int v) {
  for (int pos = 0; pos < num; pos++)
    if (ws_host[esmoe::ws_rec(pos) + kind] <= v && v < ws_host[esmoe::ws_rec(pos + 1) + kind]) return pos;
  return -1;
}
void fill_out5(int32_t* out5, int e, const esmoe::TileCoord& t) {
  out5[0] = e; out5[1] = t.mt * 16; out5[2] = t.nt * 64; out5[3] = t.m0; out5[4] = t.n0;
}
}  // namespace

int esmoe_host_decode_heavy(const int32_t* problem_sizes_host, const int32_t* ws_host, int num_experts, int n,
                            int force_bm, int kind, int xcd, int ticket, int32_t* out5) {
  g_err[0] = 0;
  if (!problem_sizes_host || !ws_host || !out5 || xcd < 0 || xcd >= esmoe::kXcds || ticket < 0)
    return fail(ESMOE_ERR_INVALID_ARGUMENT, "bad argument to esmoe_host_decode_heavy");
  const esmoe::SchedPolicy p = default_policy(force_bm, kind);
  const int blk = esmoe::sched_ticket_block(xcd, ticket);
  if (blk >= ws_host[esmoe::kWsHeavyBlocks]) return 2;   // this XCD's queue is exhausted
  const int pos = host_position(ws_host, num_experts, esmoe::kRecBlock, blk);
  if (pos < 0) return fail(ESMOE_ERR_INVALID_ARGUMENT, "workspace does not hold a schedule");
  const int32_t* rec = ws_host + esmoe::ws_rec(pos);
  esmoe::TileCoord t;
  if (!esmoe::sched_decode_heavy(blk - rec[esmoe::kRecBlock], ticket % esmoe::kBlkTiles, rec[esmoe::kRecRows], n, p, &t))
    return 1;   // ticket outside the expert's tile grid: skipped
  fill_out5(out5, rec[esmoe::kRecExpert], t);
  return 0;
}

int esmoe_host_decode_light(const int32_t* problem_sizes_host, const int32_t* ws_host, int num_experts, int n,
                            int force_bm, int kind, int item, int32_t* out5) {
  g_err[0] = 0;
  if (!problem_sizes_host || !ws_host || !out5) return fail(ESMOE_ERR_INVALID_ARGUMENT, "null pointer");
  const esmoe::SchedPolicy p = default_policy(force_bm, kind);
  if (item < 0 || item >= ws_host[esmoe::kWsLightTotal]) return fail(ESMOE_ERR_INVALID_ARGUMENT, "item out of range");
  int half = -1;
  const int idx = esmoe::sched_light_item_of_ticket(item, ws_host[esmoe::kWsLightSplit], &half);
  const int pos = host_position(ws_host, num_experts, esmoe::kRecItem, idx);
  if (pos < 0) return fail(ESMOE_ERR_INVALID_ARGUMENT, "workspace does not hold a schedule");
  const int32_t* rec = ws_host + esmoe::ws_rec(pos);
  const esmoe::TileCoord t = esmoe::sched_decode_light(idx - rec[esmoe::kRecItem], rec[esmoe::kRecRows], p, half);
  if (t.n0 >= n) return 1;   // second half of a last column tile that is 128 columns wide: skipped
  fill_out5(out5, rec[esmoe::kRecExpert], t);
  return 0;
}

const char* esmoe_last_error(void) { return g_err; }

const char* esmoe_version(void) { return "esmoe 0.3 (gfx950)"; }

}  // extern "C"
