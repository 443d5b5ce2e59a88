// Context, error reporting, device/pinned memory, copies and per-kernel timing.
#include "common.hpp"

namespace sn {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

LaunchScope::LaunchScope(sn_ctx* c, const char* n) : ctx(c) {
  if (!ctx->profiling) return;
  name = n;
  begin();
}

LaunchScope::LaunchScope(sn_ctx* c, const char* n, int m, int nn, int k) : ctx(c) {
  if (!ctx->profiling) return;
  char buf[160];
  snprintf(buf, sizeof(buf), "%s[%dx%dx%d]", n, m, nn, k);
  name = buf;
  begin();
}

void LaunchScope::begin() {
  if (ctx->pending.size() >= 8192) profile_drain(ctx);
  auto take = [&](hipEvent_t& e) {
    if (!ctx->event_pool.empty()) {
      e = ctx->event_pool.back();
      ctx->event_pool.pop_back();
      return true;
    }
    return hipEventCreate(&e) == hipSuccess;
  };
  if (!take(start) || !take(stop)) {
    start = stop = nullptr;
    return;
  }
  (void)hipEventRecord(start, ctx->stream);
}

LaunchScope::~LaunchScope() {
  if (!start) return;
  (void)hipEventRecord(stop, ctx->stream);
  ctx->pending.push_back({start, stop, name});
}

int profile_drain(sn_ctx* ctx) {
  if (ctx->pending.empty()) return SN_OK;
  SN_HIP(hipStreamSynchronize(ctx->stream));
  for (auto& p : ctx->pending) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
      auto it = ctx->profile.find(p.name);
      if (it == ctx->profile.end()) {
        ctx->profile_names.push_back(p.name);
        it = ctx->profile.emplace(p.name, ProfileEntry{}).first;
      }
      it->second.total_ms += ms;
      it->second.launches += 1;
    }
    ctx->event_pool.push_back(p.start);
    ctx->event_pool.push_back(p.stop);
  }
  ctx->pending.clear();
  return SN_OK;
}

static int seq_sync_init(sn_ctx* ctx) {
  if (ctx->seq_arrived) return SN_OK;
  unsigned* arrived = nullptr;
  int* word = nullptr;
  void* word_dev = nullptr;
  int* failed = nullptr;
  SN_HIP(hipSetDevice(ctx->device));
  hipError_t e = hipMalloc(&arrived, SEQ_COUNTERS * sizeof(unsigned));
  if (e == hipSuccess) e = hipMalloc(&failed, 256);
  if (e == hipSuccess) e = hipHostMalloc(&word, sizeof(int), hipHostMallocMapped);
  if (e == hipSuccess) {
    *word = 0;
    e = hipHostGetDevicePointer(&word_dev, word, 0);
  }
  if (e != hipSuccess) {
    if (arrived) (void)hipFree(arrived);
    if (failed) (void)hipFree(failed);
    if (word) (void)hipHostFree(word);
    return fail(SN_E_HIP, "setting up the sequence kernels' counters failed: %s", hipGetErrorString(e));
  }
  ctx->seq_arrived = arrived;
  ctx->seq_next = SEQ_COUNTERS;  // nothing cleared yet
  ctx->seq_gave_up = word;
  ctx->seq_failed_dev = failed;
  SN_TRY(launch_fill(ctx, reinterpret_cast<float*>(failed), 0.f, 64));  // all-zero bits; a kernel, not a memset node
  ctx->seq_gave_up_dev = static_cast<int*>(word_dev);
  // about a microsecond per poll: two seconds before a kernel whose neighbours never arrive gives up
  ctx->seq_spin_limit = 2000000u;
  if (const char* v = getenv("SCANET_SEQUENCE_SPIN_LIMIT")) ctx->seq_spin_limit = (unsigned)strtoul(v, nullptr, 10);
  if (const char* v = getenv("SCANET_SEQUENCE_COHERENT")) ctx->seq_force_coherent = atoi(v) != 0;
  return SN_OK;
}

int seq_sync_take(sn_ctx* ctx, int groups, unsigned** block) {
  SN_TRY(seq_sync_init(ctx));
  const int64_t need = (int64_t)(groups + 1) * SEQ_GROUP_WORDS;
  SN_REQUIRE(groups >= 1 && need <= SEQ_COUNTERS, "sequence kernel: %d row groups are more than the counter area holds", groups);
  if (ctx->seq_next + need > SEQ_COUNTERS) {  // used up: the launches that used it are ahead of this fill on the stream
    SN_TRY(launch_fill(ctx, reinterpret_cast<float*>(ctx->seq_arrived), 0.f, SEQ_COUNTERS));  // all-zero bits
    ctx->seq_next = 0;
  }
  *block = ctx->seq_arrived + ctx->seq_next;
  ctx->seq_next += need;
  return SN_OK;
}

int check_async(sn_ctx* ctx) {
  if (!ctx->seq_gave_up || *(volatile int*)ctx->seq_gave_up == 0) return SN_OK;
  *(volatile int*)ctx->seq_gave_up = 0;
  // the device's copy of the flag is cleared behind everything queued so far (a kernel, not a memset node)
  if (ctx->seq_failed_dev) (void)launch_fill(ctx, reinterpret_cast<float*>(ctx->seq_failed_dev), 0.f, 1);
  ctx->seq_disabled = true;  // something else holds compute units of this GPU: do not count on the whole grid being resident again
  return fail(SN_E_STATE, "a recurrent sequence kernel gave up waiting for its neighbour workgroups (are other processes using this GPU?): "
                          "the results of the calls since the last synchronisation are invalid");
}

static int check_ctx(sn_ctx* ctx) {
  if (!ctx || ctx->magic != CTX_MAGIC) return fail(SN_E_STATE, "invalid or destroyed context handle");
  return SN_OK;
}

}  // namespace sn

using namespace sn;

extern "C" {

const char* sn_last_error(void) { return g_error; }

int sn_ctx_create(int device, void* stream, sn_ctx** out) {
  SN_REQUIRE(out != nullptr, "sn_ctx_create: out is NULL");
  *out = nullptr;
  int count = 0;
  SN_HIP(hipGetDeviceCount(&count));
  SN_REQUIRE(device >= 0 && device < count, "device %d not present (%d visible)", device, count);
  SN_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  SN_HIP(hipGetDeviceProperties(&prop, device));
  SN_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0, "device %d is %s; this library holds gfx950 code only", device,
             prop.gcnArchName);
  SN_TRY(static_scratch_init(device));
  sn_ctx* ctx = new sn_ctx();
  ctx->magic = CTX_MAGIC;
  ctx->device = device;
  ctx->compute_units = prop.multiProcessorCount;
  ctx->profiling = false;
  if (stream) {
    ctx->stream = (hipStream_t)stream;
    ctx->owns_stream = false;
  } else {
    hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
      delete ctx;
      return fail(SN_E_HIP, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
    }
    ctx->owns_stream = true;
  }
  *out = ctx;
  return SN_OK;
}

int sn_ctx_destroy(sn_ctx* ctx) {
  SN_TRY(check_ctx(ctx));
  // models (and through them replicas) keep a pointer to the context and its stream
  if (ctx->live_models != 0) return fail(SN_E_STATE, "context still has %d live models: destroy replicas and models first", ctx->live_models);
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& p : ctx->pending) {
    (void)hipEventDestroy(p.start);
    (void)hipEventDestroy(p.stop);
  }
  for (auto e : ctx->event_pool) (void)hipEventDestroy(e);
  if (ctx->seq_arrived) (void)hipFree(ctx->seq_arrived);
  if (ctx->seq_gave_up) (void)hipHostFree(ctx->seq_gave_up);
  if (ctx->seq_failed_dev) (void)hipFree(ctx->seq_failed_dev);
  if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
  ctx->magic = 0;
  delete ctx;
  return SN_OK;
}

int sn_sync(sn_ctx* ctx) {
  SN_TRY(check_ctx(ctx));
  SN_HIP(hipStreamSynchronize(ctx->stream));
  return check_async(ctx);
}

int sn_device_info(sn_ctx* ctx, char* name, int name_cap, int64_t* hbm_bytes, int32_t* compute_units) {
  SN_TRY(check_ctx(ctx));
  hipDeviceProp_t prop;
  SN_HIP(hipGetDeviceProperties(&prop, ctx->device));
  if (name && name_cap > 0) snprintf(name, (size_t)name_cap, "%s (%s)", prop.name, prop.gcnArchName);
  if (hbm_bytes) *hbm_bytes = (int64_t)prop.totalGlobalMem;
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return SN_OK;
}

int sn_buffer_alloc(sn_ctx* ctx, size_t bytes, void** out_dev) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(out_dev != nullptr, "sn_buffer_alloc: out is NULL");
  *out_dev = nullptr;
  if (bytes == 0) return SN_OK;
  SN_HIP(hipSetDevice(ctx->device));
  SN_HIP(hipMalloc(out_dev, bytes));
  return SN_OK;
}

int sn_buffer_free(sn_ctx* ctx, void* dev) {
  SN_TRY(check_ctx(ctx));
  if (!dev) return SN_OK;
  SN_HIP(hipStreamSynchronize(ctx->stream));
  SN_HIP(hipFree(dev));
  return SN_OK;
}

int sn_host_alloc(sn_ctx* ctx, size_t bytes, void** out_host) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(out_host != nullptr, "sn_host_alloc: out is NULL");
  *out_host = nullptr;
  if (bytes == 0) return SN_OK;
  SN_HIP(hipHostMalloc(out_host, bytes, hipHostMallocDefault));
  return SN_OK;
}

int sn_host_free(sn_ctx* ctx, void* host) {
  SN_TRY(check_ctx(ctx));
  if (!host) return SN_OK;
  SN_HIP(hipStreamSynchronize(ctx->stream));
  SN_HIP(hipHostFree(host));
  return SN_OK;
}

int sn_copy_h2d(sn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes) {
  SN_TRY(check_ctx(ctx));
  if (bytes == 0) return SN_OK;
  SN_REQUIRE(dst_dev && src_host, "sn_copy_h2d: null pointer");
  SN_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
  // pageable sources are staged by the runtime before the call returns; pinned ones stay in flight
  return SN_OK;
}

int sn_copy_d2h(sn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes) {
  SN_TRY(check_ctx(ctx));
  if (bytes == 0) return SN_OK;
  SN_REQUIRE(dst_host && src_dev, "sn_copy_d2h: null pointer");
  SN_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
  SN_HIP(hipStreamSynchronize(ctx->stream));
  return check_async(ctx);
}

int sn_fill(sn_ctx* ctx, float* dst_dev, float value, int64_t n) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(dst_dev || n == 0, "sn_fill: null pointer");
  return launch_fill(ctx, dst_dev, value, n);
}

int sn_optimizer_update(sn_ctx* ctx, const sn_optimizer_desc* opt, float* w_dev, const float* g_dev, float* s0_dev, float* s1_dev,
                        float* s2_dev, int64_t n, int32_t iter) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(opt != nullptr, "sn_optimizer_update: optimizer is NULL");
  SN_REQUIRE(n >= 0, "sn_optimizer_update: negative length");
  return launch_optimizer(ctx, *opt, w_dev, g_dev, s0_dev, s1_dev, s2_dev, n, iter);
}

int sn_average(sn_ctx* ctx, const float* const* inputs_host, int32_t k, int64_t n, float* out_dev) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(inputs_host && out_dev, "sn_average: null pointer");
  SN_REQUIRE(k >= 1 && k <= SN_MAX_AVG_INPUTS, "sn_average: k must be in 1..%d, got %d", SN_MAX_AVG_INPUTS, k);
  SN_REQUIRE(n >= 0, "sn_average: negative length");
  AvgInputs in;
  for (int i = 0; i < k; ++i) {
    SN_REQUIRE(inputs_host[i] != nullptr, "sn_average: input %d is NULL", i);
    in.p[i] = inputs_host[i];
  }
  return launch_average(ctx, in, k, n, out_dev, nullptr, 0);
}

int sn_random_fill(sn_ctx* ctx, float* dst_dev, int64_t n, int32_t dist, uint64_t seed, const float* scale_host, const float* shift_host) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(dst_dev || n == 0, "sn_random_fill: null pointer");
  SN_REQUIRE(n >= 0, "sn_random_fill: negative length");
  return launch_random_fill(ctx, dst_dev, n, dist, seed, scale_host, shift_host);
}

int sn_profile_enable(sn_ctx* ctx, int32_t on) {
  SN_TRY(check_ctx(ctx));
  if (!on) {
    SN_TRY(profile_drain(ctx));
    SN_TRY(check_async(ctx));
  }
  ctx->profiling = on != 0;
  return SN_OK;
}

int sn_profile_reset(sn_ctx* ctx) {
  SN_TRY(check_ctx(ctx));
  SN_TRY(profile_drain(ctx));
  SN_TRY(check_async(ctx));  // the drain synchronised the stream
  ctx->profile.clear();
  ctx->profile_names.clear();
  return SN_OK;
}

int sn_profile_count(sn_ctx* ctx, int32_t* n) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(n != nullptr, "sn_profile_count: out is NULL");
  SN_TRY(profile_drain(ctx));
  SN_TRY(check_async(ctx));  // the drain synchronised the stream
  *n = (int32_t)ctx->profile_names.size();
  return SN_OK;
}

int sn_profile_get(sn_ctx* ctx, int32_t index, char* name, int32_t name_cap, double* total_ms, int64_t* launches) {
  SN_TRY(check_ctx(ctx));
  SN_REQUIRE(index >= 0 && index < (int32_t)ctx->profile_names.size(), "sn_profile_get: index %d out of range", index);
  const std::string& key = ctx->profile_names[index];
  const ProfileEntry& e = ctx->profile[key];
  if (name && name_cap > 0) snprintf(name, (size_t)name_cap, "%s", key.c_str());
  if (total_ms) *total_ms = e.total_ms;
  if (launches) *launches = e.launches;
  return SN_OK;
}

}  // extern "C"
