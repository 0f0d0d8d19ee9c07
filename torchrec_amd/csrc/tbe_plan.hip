// Host side of the TBE lookup: plan construction (tra_tbe_create) and launch
// (tra_tbe_forward), plus the small library-level entry points.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <tuple>
#include <memory>
#include <mutex>
#include <string>

#include "tbe_lookup_impl.h"

namespace tra {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("%s: %s", what, hipGetErrorString(e));
  return TRA_ERR_HIP;
}

// Explicit specializations live in tbe_lookup_<dtype>.hip.
template <>
int launch_lookup<TRA_INT8>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_INT4>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_INT2>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_INT8 + kSplitHeader>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_INT4 + kSplitHeader>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_INT2 + kSplitHeader>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_FP16>(const LookupArgs&, int, const LaunchParams&, hipStream_t);
template <>
int launch_lookup<TRA_FP32>(const LookupArgs&, int, const LaunchParams&, hipStream_t);

// Launch shape of the pooled kernels.  Defaults are chosen from the problem
// size when a plan first sees a (batch size, route) pair and are remembered in
// the plan.  The tuning overrides (environment TRA_BALANCED, TRA_WINDOW,
// TRA_UNROLL, TRA_LDS, TRA_XCD, TRA_COST_FLOOR, TRA_FUSED_SCAN, TRA_CB) are read
// once, when the library is loaded; tra_set_tuning changes them afterwards
// (experiments and tests).  A forward never reads the environment.
struct Tuning {
  int balanced;  // 1: tbe_pooled_cu_kernel, one block per CU-sized window of bags
  int window;    // bags per block (0: derive from the problem size)
  int unroll;
  int lds_bytes;
};

struct Overrides {
  int balanced = -1;    // -1: decide by size
  int window = -1;      // <= 0: derive
  int unroll = -1;
  int lds = -1;
  int xcd = -1;         // 0: no XCD remap of the window kernel's blocks
  int cost_floor = -1;
  int fused_scan = -1;  // -1: decide by size
  int cb = -1;          // smaller lane chunks (plan creation)
  int fork = -1;        // 0: the launches of a multi-class call stay on the caller's stream
};

static int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : fallback;
}

static Overrides overrides_from_env() {
  Overrides o;
  o.balanced = env_int("TRA_BALANCED", -1);
  o.window = env_int("TRA_WINDOW", -1);
  o.unroll = env_int("TRA_UNROLL", -1);
  o.lds = env_int("TRA_LDS", -1);
  o.xcd = env_int("TRA_XCD", -1);
  o.cost_floor = env_int("TRA_COST_FLOOR", -1);
  o.fused_scan = env_int("TRA_FUSED_SCAN", -1);
  o.cb = env_int("TRA_CB", -1);
  o.fork = env_int("TRA_FORK", -1);
  return o;
}

static Overrides g_ovr = overrides_from_env();
// Bumped by tra_set_tuning: launch geometry remembered under an older value is recomputed.
static std::atomic<int> g_ovr_gen{0};

static Tuning choose_tuning(int num_cus, int64_t bags, int64_t num_indices) {
  Tuning t;
  // Ranking bags by length pays once every CU gets a few dozen bags (measured
  // crossover on 26 int4 tables: between 6.6k bags / 130k ids and 13k / 260k).
  t.balanced = bags >= 40 * (int64_t)num_cus && num_indices >= 640 * (int64_t)num_cus;
  t.window = 0;
  t.unroll = 4;
  t.lds_bytes = 48 * 1024;  // with the static arrays > half of a CU's LDS: one block per CU
  if (g_ovr.balanced >= 0) t.balanced = g_ovr.balanced;
  if (g_ovr.window >= 0) t.window = g_ovr.window;
  if (g_ovr.unroll >= 0) t.unroll = g_ovr.unroll;
  if (g_ovr.lds >= 0) t.lds_bytes = g_ovr.lds;
  if (t.window > kMaxWindow) t.window = kMaxWindow;
  if (t.window < 0) t.window = 0;
  return t;
}

}  // namespace tra

// Scratch of tra_tbe_forward_lengths_static: the offsets array and the scan's
// tile sums of one call.  One copy per GPU, held until the process ends.
constexpr int64_t kStaticScratchBytes = 8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace tra {

// Device address of `scratch` on each GPU (the array's name is only a host-side
// handle).  Resolved when the first plan is created on a device, that device
// being current.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

static int resolve_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices) {
    set_error("device index %d is beyond the %d devices the library tracks", device, kMaxDevices);
    return TRA_ERR_TOO_LARGE;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] != nullptr) return TRA_OK;
  void* p = nullptr;
  hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
  if (p == nullptr || (uintptr_t)p % 256 != 0) {
    set_error("static scratch resolved to %p (expected a 256-byte aligned device address)", p);
    return TRA_ERR_HIP;
  }
  g_scratch_ptr[device] = p;
  return TRA_OK;
}

}  // namespace tra

using namespace tra;

// Launch geometry of one launch class for one (batch size, route).
struct ClassGeometry {
  SubClass sub[kMaxSub];
  int n_sub = 0;
  int grid = 0;
  int xcd_blocks = 0;
  int xcd_count = 1;
};

// What a plan remembers about a call shape it has seen: the route and, per
// launch class, the grid and windows.  Recomputed when the tuning overrides change.
struct Geometry {
  int32_t batch_size = -1;
  int64_t nobag_indices = -1;  // sequence lookups size their grid by the id count
  int balanced = 0;
  int nobag = 0;
  int gen = -1;
  Tuning tune{};
  std::vector<ClassGeometry> cls;
};

constexpr int kGeometrySlots = 8;

// A call of at least this many launch classes runs them on two streams (see forward_impl).  The
// fork and the join cost about 10 us of dependencies between queues, every pair of neighbouring
// launches gains a few: with launches of 25 - 30 us each, two classes lose 11 %, three and four
// are even (-1 %, +0.5 %), five gain 8 %, seven (of about 50 us) 9 %.
constexpr size_t kForkMinClasses = 5;

struct tra_tbe {
  int device = 0;
  int num_cus = 256;  // compute units of the device (hipDeviceProp_t::multiProcessorCount)
  int num_xcd = 8;    // accelerator dies, each with its own L2 (hipDeviceAttributeNumberOfXccs)
  int num_features = 0;
  bool same_dim = true;  // every feature has the same dim (required for POOL_NONE)
  int dim0 = 0;
  int max_key_pos = 0;          // largest feature position among the input keys
  size_t max_class_feats = 0;   // features of the largest launch class
  std::vector<FeatureDesc> slices;  // host copy
  FeatureDesc* slices_dev = nullptr;
  int32_t* feats_dev = nullptr;  // all classes' slice lists, concatenated
  FeatureDesc* cdescs_dev = nullptr;  // the descriptors in that order: cdescs[i] = slices[feats[i]]
  unsigned long long* err_dev = nullptr;
  void* static_scratch = nullptr;  // this device's copy of the library's static scratch array
  std::atomic<int> bad_to_row0{0};  // 1: ids outside their table pool row 0 (tra_tbe_set_bounds_check_mode)
  // The second stream of a multi-class call (plans of kForkMinClasses launch classes or more; default
  // priority), the events that fork it from and join it to the caller's stream, and which of the
  // two streams every class is launched on, in launch order (largest class first).
  std::mutex fork_mutex;
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr;
  hipEvent_t ev_join = nullptr;
  std::vector<int> launch_order;     // class indices
  std::vector<uint8_t> on_side;      // per class index: 1 = launched on `side`
  std::vector<LaunchClass> classes;
  std::vector<LookupArgs> base_args;  // per class: everything a call does not change
  std::mutex geo_mutex;
  std::shared_ptr<const Geometry> geo[kGeometrySlots];
  int geo_next = 0;
};

extern "C" {

int tra_version(void) { return 1; }

const char* tra_last_error(void) { return g_err; }

int tra_device_arch(char* buf, int buf_len) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    set_error("no HIP device");
    return TRA_ERR_NO_DEVICE;
  }
  int dev = 0;
  TRA_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  TRA_HIP(hipGetDeviceProperties(&prop, dev));
  if (buf && buf_len > 0) {
    strncpy(buf, prop.gcnArchName, (size_t)buf_len - 1);
    buf[buf_len - 1] = 0;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error("device arch %s is not gfx950", prop.gcnArchName);
    return TRA_ERR_NO_DEVICE;
  }
  return TRA_OK;
}

int tra_set_tuning(const char* name, int32_t value) {
  if (!name) {
    set_error("tra_set_tuning: null name");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  struct { const char* n; int* v; } const knobs[] = {
      {"balanced", &g_ovr.balanced}, {"window", &g_ovr.window}, {"unroll", &g_ovr.unroll},
      {"lds", &g_ovr.lds}, {"xcd", &g_ovr.xcd}, {"cost_floor", &g_ovr.cost_floor},
      {"fused_scan", &g_ovr.fused_scan}, {"cb", &g_ovr.cb}, {"fork", &g_ovr.fork}};
  for (const auto& k : knobs)
    if (strcmp(name, k.n) == 0) {
      *k.v = value < 0 ? -1 : value;
      g_ovr_gen.fetch_add(1, std::memory_order_relaxed);
      return TRA_OK;
    }
  set_error("tra_set_tuning: unknown knob '%s'", name);
  return TRA_ERR_INVALID_ARGUMENT;
}

int tra_tbe_create(const tra_table_spec* tables, int32_t num_tables,
                   const int32_t* feature_table_map, const int32_t* feature_positions,
                   int32_t num_features, tra_tbe_t* out) {
  if (!out || num_tables < 0 || num_features < 0 || (num_tables > 0 && !tables) ||
      (num_features > 0 && !feature_table_map)) {
    set_error("tra_tbe_create: null or negative argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  *out = nullptr;
  for (int t = 0; t < num_tables; ++t) {
    const tra_table_spec& s = tables[t];
    const int bits = bits_of(s.dtype);
    if (bits == 0) {
      set_error("table %d: unsupported dtype %d", t, s.dtype);
      return TRA_ERR_INVALID_ARGUMENT;
    }
    if (s.rows < 1) {
      // Skipped ids are redirected to row 0, so every table needs one.
      set_error("table %d has no rows", t);
      return TRA_ERR_INVALID_ARGUMENT;
    }
    if (s.dim <= 0 || (int64_t)s.dim * bits % 32 != 0) {
      set_error("table %d: dim %d with %d-bit elements is not a whole number of dwords", t,
                s.dim, bits);
      return TRA_ERR_INVALID_ARGUMENT;
    }
    const int need = s.dim * bits / 8 + header_bytes(s.dtype);
    if (s.row_bytes < need || s.row_bytes % 4 != 0 || s.offset % 4 != 0 || s.offset < 0) {
      set_error("table %d: row_bytes %d (need >= %d) and offset must be multiples of 4", t,
                s.row_bytes, need);
      return TRA_ERR_INVALID_ARGUMENT;
    }
  }
  auto plan = new tra_tbe();
  plan->num_features = num_features;
  int col = 0;
  // (dtype, cb, rows cut into several slices) -> slice ids
  std::map<std::tuple<int, int, int>, std::vector<int>> by_class;
  std::vector<int> slice_lpr;
  for (int f = 0; f < num_features; ++f) {
    const int t = feature_table_map[f];
    if (t < 0 || t >= num_tables || (feature_positions && feature_positions[f] < 0)) {
      delete plan;
      set_error("feature %d maps to table %d of %d (or has a negative position)", f, t,
                num_tables);
      return TRA_ERR_INVALID_ARGUMENT;
    }
    const tra_table_spec& s = tables[t];
    if (f == 0) plan->dim0 = s.dim;
    if (s.dim != plan->dim0) plan->same_dim = false;
    const int bits = bits_of(s.dtype);
    const int payload = s.dim * bits / 8;
    // Bytes per lane.  Rows of up to 64 payload bytes take 8-byte chunks: with
    // 16-byte chunks a wave would gather from 16-64 different rows per load,
    // which measured 9 % slower on the mixed-width workload (and 3 % faster on
    // the all-64-byte one).
    int cb = payload % 16 == 0 && payload > 64 ? 16 : (payload % 8 == 0 ? 8 : 4);
    {
      const int force = g_ovr.cb;  // tuning: smaller lane chunks, or 16 bytes wherever they divide the row
      if ((force == 8 || force == 4) && force < cb && payload % force == 0) cb = force;
      if (force == 16 && payload % 16 == 0) cb = 16;
    }
    const int max_slice = cb * kWaveSize;  // bytes one wave-wide lane group covers
    // A row with a header whose lanes take 8 or 4 bytes normally gets its header with the
    // first lane's chunk; cut into several slices, only the first slice could, so all its
    // slices go to a launch class of their own that loads the header separately.
    const int split = payload > max_slice && header_bytes(s.dtype) != 0 && cb <= 8 ? 1 : 0;
    for (int off = 0; off < payload; off += max_slice) {
      const int bytes = std::min(max_slice, payload - off);
      FeatureDesc d;
      d.table_offset = s.offset;
      d.rows = s.rows;
      d.dim = s.dim;
      d.row_bytes = s.row_bytes;
      d.out_col = col + off * 8 / bits;
      d.dtype = s.dtype;
      d.feature = feature_positions ? feature_positions[f] : f;
      d.payload_off = off;
      by_class[{s.dtype, cb, split}].push_back((int)plan->slices.size());
      plan->slices.push_back(d);
      slice_lpr.push_back(bytes / cb);
    }
    col += s.dim;
  }
  // Classes: slices sorted by lanes-per-row; at most kMaxSub distinct values each.
  std::vector<int32_t> all_feats;
  for (auto& kv : by_class) {
    std::vector<int>& ids = kv.second;
    std::stable_sort(ids.begin(), ids.end(),
                     [&](int x, int y) { return slice_lpr[x] < slice_lpr[y]; });
    LaunchClass cur;
    int distinct = 0, last_lpr = -1;
    auto flush = [&]() {
      if (!cur.feats.empty()) plan->classes.push_back(cur);
      cur = LaunchClass();
      distinct = 0;
      last_lpr = -1;
    };
    for (int id : ids) {
      if (slice_lpr[id] != last_lpr) {
        if (distinct == kMaxSub) flush();
        ++distinct;
        last_lpr = slice_lpr[id];
      }
      cur.dtype = std::get<0>(kv.first);
      cur.cb = std::get<1>(kv.first);
      cur.split = std::get<2>(kv.first) != 0;
      cur.feats.push_back(id);
      cur.lprs.push_back(slice_lpr[id]);
    }
    flush();
  }
  hipError_t e = hipGetDevice(&plan->device);
  if (e == hipSuccess) {
    // The window kernel sizes its grid by the CU count and keeps consecutive
    // windows on one die: both come from the device, so a partitioned GPU
    // (fewer CUs, fewer dies) gets a launch that fits it.
    int cus = 0, xcds = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, plan->device);
    if (e == hipSuccess && hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, plan->device) != hipSuccess) {
      (void)hipGetLastError();
      xcds = 1;
    }
    if (e == hipSuccess) {
      if (cus < 1) {
        delete plan;
        set_error("tra_tbe_create: device reports %d compute units", cus);
        return TRA_ERR_NO_DEVICE;
      }
      plan->num_cus = cus;
      // Blocks are dealt to the dies round-robin; the remap assumes every die
      // has the same number of CUs.  Anything else: no remap.
      plan->num_xcd = (xcds >= 1 && cus % xcds == 0) ? xcds : 1;
      // Only tra_tbe_forward_lengths_static needs the static scratch: where it cannot be
      // resolved the plan is still good for every other entry point, and that one reports it.
      if (resolve_static_scratch(plan->device) == TRA_OK) {
        plan->static_scratch = g_scratch_ptr[plan->device];
      } else {
        (void)hipGetLastError();
        plan->static_scratch = nullptr;
      }
    }
  }
  size_t total = 0;
  for (auto& c : plan->classes) total += c.feats.size();
  if (e == hipSuccess && !plan->slices.empty()) {
    e = hipMalloc((void**)&plan->slices_dev, plan->slices.size() * sizeof(FeatureDesc));
    if (e == hipSuccess)
      e = hipMemcpy(plan->slices_dev, plan->slices.data(),
                    plan->slices.size() * sizeof(FeatureDesc), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&plan->feats_dev, total * sizeof(int32_t));
    if (e == hipSuccess) {
      size_t pos = 0;
      for (auto& c : plan->classes) {
        c.feats_dev = plan->feats_dev + pos;
        all_feats.insert(all_feats.end(), c.feats.begin(), c.feats.end());
        pos += c.feats.size();
      }
      e = hipMemcpy(plan->feats_dev, all_feats.data(), total * sizeof(int32_t),
                    hipMemcpyHostToDevice);
    }
    if (e == hipSuccess) e = hipMalloc((void**)&plan->cdescs_dev, total * sizeof(FeatureDesc));
    if (e == hipSuccess) {
      std::vector<FeatureDesc> ordered;
      for (int32_t id : all_feats) ordered.push_back(plan->slices[id]);
      e = hipMemcpy(plan->cdescs_dev, ordered.data(), total * sizeof(FeatureDesc), hipMemcpyHostToDevice);
    }
  }
  if (e == hipSuccess) e = hipMalloc((void**)&plan->err_dev, sizeof(unsigned long long));
  if (e == hipSuccess) e = hipMemset(plan->err_dev, 0, sizeof(unsigned long long));
  if (e != hipSuccess) {
    tra_tbe_destroy(plan);
    return hip_fail(e, "tra_tbe_create");
  }
  for (const FeatureDesc& d : plan->slices) plan->max_key_pos = std::max(plan->max_key_pos, (int)d.feature);
  for (LaunchClass& cls : plan->classes) {
    for (int id : cls.feats) {
      cls.cols_aligned_fp16 = cls.cols_aligned_fp16 && (int64_t)plan->slices[id].out_col * 2 % 16 == 0;
      cls.cols_aligned_fp32 = cls.cols_aligned_fp32 && (int64_t)plan->slices[id].out_col * 4 % 16 == 0;
    }
    plan->max_class_feats = std::max(plan->max_class_feats, cls.feats.size());
    LookupArgs a;
    memset(&a, 0, sizeof(a));
    a.descs = plan->slices_dev;
    a.feats = cls.feats_dev;
    a.cdescs = plan->cdescs_dev + (cls.feats_dev - plan->feats_dev);
    a.err_count = plan->err_dev;
    for (size_t i = 0; i < cls.feats.size() && i < (size_t)kMaxPos; ++i)
      a.feat_pos[i] = (int16_t)plan->slices[cls.feats[i]].feature;
    plan->base_args.push_back(a);
  }
  // Launch order and streams.  The launches of a call write disjoint output columns, so they may
  // overlap.  A launch leaves compute units idle before its first rows arrive and while its last
  // blocks finish; with consecutive launches on alternating streams the next launch's blocks fill
  // them.  Measured on 7 classes (64 mixed tables, 7.9 M ids): 379 us on one stream, 345 us on two
  // with the largest class first (348 us in plan order, 347 us smallest first, 355 us with the
  // classes dealt to the two streams by balanced work, where neighbours often share a stream), 376
  // and 385 us on three and four streams.  A class's work is taken as 128-byte lines per row,
  // summed over its features.
  {
    const size_t nc = plan->classes.size();
    std::vector<double> cost(nc, 0.0);
    for (size_t ci = 0; ci < nc; ++ci)
      for (int32_t lpr : plan->classes[ci].lprs)
        cost[ci] += std::max(1.0, std::ceil((double)lpr * plan->classes[ci].cb / 128.0));
    plan->launch_order.resize(nc);
    for (size_t ci = 0; ci < nc; ++ci) plan->launch_order[ci] = (int)ci;
    plan->on_side.assign(nc, 0);
    // (tuning: `fork` = k > 1 at plan creation lowers or raises the class count from which a plan forks)
    const size_t fork_min = g_ovr.fork > 1 ? (size_t)g_ovr.fork : kForkMinClasses;
    if (nc >= fork_min) {
      std::stable_sort(plan->launch_order.begin(), plan->launch_order.end(),
                       [&](int x, int y) { return cost[x] > cost[y]; });
      for (size_t k = 0; k < nc; ++k) plan->on_side[plan->launch_order[k]] = (uint8_t)(k & 1);
      if (hipStreamCreateWithFlags(&plan->side, hipStreamNonBlocking) != hipSuccess ||
          hipEventCreateWithFlags(&plan->ev_fork, hipEventDisableTiming) != hipSuccess ||
          hipEventCreateWithFlags(&plan->ev_join, hipEventDisableTiming) != hipSuccess) {
        const int rc = hip_fail(hipGetLastError(), "creating the second stream of a multi-class plan");
        tra_tbe_destroy(plan);
        return rc;
      }
    }
  }
  *out = plan;
  return TRA_OK;
}

int tra_tbe_destroy(tra_tbe_t tbe) {
  if (!tbe) return TRA_OK;
  if (tbe->slices_dev) (void)hipFree(tbe->slices_dev);
  if (tbe->feats_dev) (void)hipFree(tbe->feats_dev);
  if (tbe->cdescs_dev) (void)hipFree(tbe->cdescs_dev);
  if (tbe->err_dev) (void)hipFree(tbe->err_dev);
  if (tbe->side) (void)hipStreamDestroy(tbe->side);
  if (tbe->ev_join) (void)hipEventDestroy(tbe->ev_join);
  if (tbe->ev_fork) (void)hipEventDestroy(tbe->ev_fork);
  delete tbe;
  return TRA_OK;
}

// Whether a pooled call goes to the per-CU window kernel: the size heuristic
// (or its override) and the limits of the kernel's packed window entries.
static bool use_window_kernel(const tra_tbe* tbe, const Tuning& tune, bool nobag,
                              int32_t batch_size) {
  return !nobag && tune.balanced && batch_size <= (1 << kBagBits) && tbe->max_key_pos <= 32767 &&
         (int64_t)tbe->max_class_feats < (int64_t(1) << (32 - kBagBits)) &&
         (int64_t)tbe->max_class_feats * batch_size < (int64_t(1) << 31);
}

// Largest number of features one window of the from-lengths kernel may span.
constexpr int kMaxWindowFeatures = 32;

// Can a pooled call with these sizes take the window kernel in its
// from-lengths form (which needs no offsets)?
static bool fused_scan_possible(const tra_tbe* tbe, int32_t batch_size, int32_t num_keys,
                                int64_t num_indices, int32_t pooling_mode, const void* lengths) {
  if (pooling_mode == TRA_POOL_NONE || batch_size <= 0 || tbe->num_features == 0) return false;
  if ((uintptr_t)lengths % 16 != 0) return false;
  const Tuning tune = choose_tuning(tbe->num_cus, (int64_t)tbe->num_features * batch_size, num_indices);
  if (!use_window_kernel(tbe, tune, false, batch_size)) return false;
  const int fused = g_ovr.fused_scan;
  if (fused >= 0) return fused != 0;
  // A window of up to kMaxWindow bags spans kMaxWindow / B + 2 features at most.
  if (kMaxWindow / batch_size + 2 > kMaxWindowFeatures) return false;
  // Every block of every launch sums the lengths in front of its window
  // (about 1.3 us + 1 us per 40k lengths, measured); a separate scan costs
  // about 7 us once.  Take whichever is less.
  const int64_t n = (int64_t)num_keys * batch_size;
  return (int64_t)tbe->classes.size() * (13 + n / 4000) < 70;
}

// A pooled call too small for the window kernel whose lengths are few enough
// that every block of the static kernel can sum the ones in front of its bags
// itself: one launch instead of a scan and a lookup.
constexpr int64_t kSmallFusedMaxLengths = 16384;

static bool small_fused_scan_possible(const tra_tbe* tbe, int32_t batch_size, int32_t num_keys,
                                      int64_t num_indices, int32_t pooling_mode, const void* lengths) {
  if (pooling_mode == TRA_POOL_NONE || batch_size <= 0 || tbe->num_features == 0) return false;
  if ((uintptr_t)lengths % 16 != 0 || g_ovr.fused_scan == 0) return false;
  const Tuning tune = choose_tuning(tbe->num_cus, (int64_t)tbe->num_features * batch_size, num_indices);
  if (use_window_kernel(tbe, tune, false, batch_size)) return false;
  return (int64_t)num_keys * batch_size <= kSmallFusedMaxLengths;
}

int tra_tbe_launch_info(tra_tbe_t tbe, int32_t batch_size, int64_t num_indices,
                        int32_t pooling_mode, int32_t lengths_num_keys, char* buf,
                        int32_t buf_len) {
  if (!tbe || !buf || buf_len <= 0) {
    set_error("tra_tbe_launch_info: null argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const bool nobag = pooling_mode == TRA_POOL_NONE;
  const Tuning tune = choose_tuning(tbe->num_cus, (int64_t)tbe->num_features * batch_size, num_indices);
  const bool balanced = use_window_kernel(tbe, tune, nobag, batch_size);
  // lengths entry point: same decision as tra_tbe_forward_lengths (aligned lengths assumed)
  const bool fused = lengths_num_keys > 0 &&
                     (fused_scan_possible(tbe, batch_size, lengths_num_keys, num_indices, pooling_mode,
                                          (const void*)16) ||
                      small_fused_scan_possible(tbe, batch_size, lengths_num_keys, num_indices, pooling_mode,
                                                (const void*)16));
  static const char* const kDtypeName[] = {"fp32", "fp16", "int8", "int4", "int2"};
  std::string text;
  // In launch order; a plan with a second stream alternates between the two.
  const bool two_streams = tbe->side != nullptr && balanced && g_ovr.fork != 0;
  for (const int ci : tbe->launch_order) {
    const LaunchClass& cls = tbe->classes[ci];
    char line[200];
    snprintf(line, sizeof(line), "%s%s dtype=%s lane_bytes=%d slices=%d%s%s",
             text.empty() ? "" : "; ",
             nobag ? "tbe_nobag_kernel" : (balanced ? "tbe_pooled_cu_kernel" : "tbe_pooled_kernel"),
             kDtypeName[cls.dtype], cls.cb, (int)cls.feats.size(),
             two_streams ? (tbe->on_side[ci] ? " on the plan's second stream" : " on the caller's stream") : "",
             fused ? " from_lengths" : "");
    text += line;
  }
  if (lengths_num_keys > 0 && !fused) text = "scan_small_kernel or tile_sums_kernel + scan_tiles_kernel; " + text;
  snprintf(buf, (size_t)buf_len, "%s", text.c_str());
  return TRA_OK;
}

// Position weights of a call: one fp32 vector per input key, concatenated on
// the device; key_start / key_len (host) say where key p's vector sits.
struct PositionWeights {
  const float* table;
  int64_t table_len;
  const int32_t* key_start;
  const int32_t* key_len;
  int32_t num_keys;
};

// Grid and windows of every launch class for one call shape.
static void compute_geometry(const tra_tbe* tbe, const Tuning& tune, bool balanced, bool nobag,
                             int32_t batch_size, int64_t num_indices, Geometry& g) {
  const int num_cus = tbe->num_cus;
  g.batch_size = batch_size;
  g.nobag_indices = nobag ? num_indices : -1;
  g.balanced = balanced ? 1 : 0;
  g.nobag = nobag ? 1 : 0;
  g.tune = tune;
  g.cls.assign(tbe->classes.size(), ClassGeometry());
  for (size_t ci = 0; ci < tbe->classes.size(); ++ci) {
    const LaunchClass& cls = tbe->classes[ci];
    ClassGeometry& cg = g.cls[ci];
    // Window kernel: every block should get about the same amount of work, so
    // a sub-class's window (bags per block) shrinks with its row width.  A
    // row costs its payload bytes, but never less than 256: below that the
    // per-row requests (id, header, one line) dominate and rows of any width
    // take the same time.  Aim at one block per CU; more passes when a window
    // would not fit the kernel's LDS arrays.
    const int64_t cost_floor = g_ovr.cost_floor >= 0 ? g_ovr.cost_floor : 256;
    auto bag_cost = [&](size_t i) { return std::max<int64_t>((int64_t)cls.lprs[i] * cls.cb, cost_floor); };
    int64_t work_per_block = 0;
    if (balanced) {
      int64_t total = 0, min_cost = INT64_MAX;
      for (size_t i = 0; i < cls.feats.size(); ++i) {
        total += (int64_t)batch_size * bag_cost(i);
        min_cost = std::min(min_cost, bag_cost(i));
      }
      int64_t blocks = num_cus;
      while ((total + blocks - 1) / blocks > (int64_t)kMaxWindow * min_cost) blocks += num_cus;
      work_per_block = (total + blocks - 1) / blocks;
      // Rounding each sub-class up to whole windows must not spill a few
      // blocks into an extra pass: grow the share until the grid fits.
      for (int iter = 0; iter < 64; ++iter) {
        int64_t grid = 0;
        for (size_t i = 0; i < cls.feats.size();) {
          size_t j = i;
          while (j < cls.feats.size() && cls.lprs[j] == cls.lprs[i]) ++j;
          const int64_t w = std::max<int64_t>(
              64, std::min<int64_t>((work_per_block + bag_cost(i) - 1) / bag_cost(i), kMaxWindow));
          grid += ((int64_t)(j - i) * batch_size + w - 1) / w;
          i = j;
        }
        if (grid <= blocks) break;
        work_per_block += std::max<int64_t>(1, work_per_block / 128);
      }
    }
    int grid = 0;
    int n_sub = 0;
    for (size_t i = 0; i < cls.feats.size();) {
      size_t j = i;
      while (j < cls.feats.size() && cls.lprs[j] == cls.lprs[i]) ++j;
      SubClass& sc = cg.sub[n_sub++];
      sc.first = (int)i;
      sc.count = (int)(j - i);
      sc.lpr = cls.lprs[i];
      sc.key0 = tbe->slices[cls.feats[i]].feature;
      for (size_t k = i; k < j; ++k)
        if (tbe->slices[cls.feats[k]].feature != sc.key0 + (int)(k - i)) sc.key0 = -1;
      const int gpw = kWaveSize / sc.lpr;
      const int per_block = kWavesPerBlock * gpw;
      sc.tile_start = grid;
      if (nobag) {
        // Blocks stride over a feature's ids; enough blocks for ~the average
        // feature, capped so the grid stays modest.
        int64_t avg = num_indices > 0 ? num_indices / tbe->num_features + 1 : 4096;
        int64_t t = (avg + per_block - 1) / per_block;
        sc.tiles_per_feat = (int)std::max<int64_t>(1, std::min<int64_t>(t, 8192));
        grid += sc.count * sc.tiles_per_feat;
      } else if (balanced) {
        const int64_t nb = (int64_t)sc.count * batch_size;
        int64_t window = tune.window > 0 ? tune.window : (work_per_block + bag_cost(i) - 1) / bag_cost(i);
        window = std::max<int64_t>(64, std::min<int64_t>(window, kMaxWindow));
        sc.tiles_per_feat = 0;
        sc.window = (int)window;
        grid += (int)((nb + window - 1) / window);
      } else {
        sc.tiles_per_feat = (batch_size + per_block - 1) / per_block;
        grid += sc.count * sc.tiles_per_feat;
      }
      i = j;
    }
    cg.n_sub = n_sub;
    cg.grid = grid;
    cg.xcd_count = 1;
    cg.xcd_blocks = 0;
    if (balanced) {
      // The XCD remap needs a grid that is a whole number of blocks per die
      // (surplus blocks exit at once).
      const int nx = tbe->num_xcd;
      cg.grid = (grid + nx - 1) / nx * nx;
      if (nx > 1 && g_ovr.xcd != 0) {
        cg.xcd_blocks = cg.grid / nx;
        cg.xcd_count = nx;
      }
    }
  }
}

// The grid of a sequence lookup follows the number of ids, which differs from call to call in
// service.  Geometries are kept per id count rounded up to a step of an eighth of its power of
// two (the blocks of a feature stride over its ids, so any grid of about the right size will
// do): neighbouring batch sizes share an entry instead of each evicting one.
static int64_t quantized_id_count(int64_t n) {
  if (n <= 1024) return 1024;
  int lg = 0;
  while ((int64_t(1) << (lg + 1)) <= n) ++lg;
  const int64_t step = int64_t(1) << (lg - 3);
  return (n + step - 1) / step * step;
}

static int forward_impl(tra_tbe_t tbe, const void* weights, const void* indices,
                        const void* offsets, bool from_lengths, int32_t idx_is_i64,
                        const float* per_sample_weights, int32_t batch_size, int64_t num_indices,
                        int32_t pooling_mode, int32_t out_dtype, void* out, int64_t out_stride,
                        void* stream, const PositionWeights* pw = nullptr, bool one_stream = false) {
  if (!tbe) {
    set_error("tra_tbe_forward: null plan");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (pooling_mode != TRA_POOL_SUM && pooling_mode != TRA_POOL_MEAN &&
      pooling_mode != TRA_POOL_NONE) {
    set_error("tra_tbe_forward: bad pooling mode %d", pooling_mode);
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (out_dtype != TRA_FP32 && out_dtype != TRA_FP16) {
    set_error("tra_tbe_forward: output dtype %d is not fp32/fp16", out_dtype);
    return TRA_ERR_UNSUPPORTED;
  }
  if (batch_size < 0) {
    set_error("tra_tbe_forward: negative batch size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const bool nobag = pooling_mode == TRA_POOL_NONE;
  if (tbe->num_features == 0 || batch_size == 0 || (nobag && num_indices == 0)) return TRA_OK;
  if (num_indices < 0) {
    set_error("tra_tbe_forward: num_indices is required");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (!weights || !offsets || !out || (!indices && num_indices != 0)) {
    set_error("tra_tbe_forward: null buffer");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  {
    // Rows are read as dwords; ids, bag boundaries and weights as whole elements.
    const uintptr_t isz = idx_is_i64 ? 8 : 4;
    if ((uintptr_t)weights % 4 != 0 || (uintptr_t)indices % isz != 0 ||
        (uintptr_t)offsets % isz != 0 || (uintptr_t)per_sample_weights % 4 != 0 ||
        (uintptr_t)out % (out_dtype == TRA_FP16 ? 2 : 4) != 0 ||
        (pw != nullptr && (uintptr_t)pw->table % 4 != 0)) {
      set_error("tra_tbe_forward: a buffer is not aligned to its element size");
      return TRA_ERR_INVALID_ARGUMENT;
    }
  }
  if (nobag && !tbe->same_dim) {
    set_error("tra_tbe_forward: sequence lookup needs one embedding dim for all tables");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  {
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != tbe->device) {
      set_error("tra_tbe_forward: plan was created on device %d, current device is %d", tbe->device,
                cur);
      return TRA_ERR_INVALID_ARGUMENT;
    }
  }
  const int esz = out_dtype == TRA_FP16 ? 2 : 4;
  hipStream_t s = (hipStream_t)stream;
  // Route and launch geometry: remembered per (batch size, route) in the plan.
  std::shared_ptr<const Geometry> geo;
  {
    std::lock_guard<std::mutex> lock(tbe->geo_mutex);
    const int gen = g_ovr_gen.load(std::memory_order_relaxed);
    const Tuning tune = choose_tuning(tbe->num_cus, (int64_t)tbe->num_features * batch_size, num_indices);
    const int balanced = use_window_kernel(tbe, tune, nobag, batch_size) ? 1 : 0;
    const int64_t geo_indices = nobag ? quantized_id_count(num_indices) : num_indices;
    for (const auto& g : tbe->geo)
      if (g && g->batch_size == batch_size && g->gen == gen && g->balanced == balanced &&
          g->nobag == (int)nobag && (!nobag || g->nobag_indices == geo_indices)) {
        geo = g;
        break;
      }
    if (!geo) {
      auto g = std::make_shared<Geometry>();
      compute_geometry(tbe, tune, balanced != 0, nobag, batch_size, geo_indices, *g);
      g->gen = gen;
      geo = g;
      tbe->geo[tbe->geo_next] = geo;  // a call still launching from the replaced entry keeps it alive
      tbe->geo_next = (tbe->geo_next + 1) % kGeometrySlots;
    }
  }
  const Geometry& geo_local = *geo;
  const bool balanced = geo_local.balanced != 0;
  // A call of several launch classes runs them on two streams: the caller's stream forks into the
  // plan's second stream before the first launch and joins it after the last.  One call at a time
  // per plan enqueues such a sequence (the events are the plan's).  Not while the caller's stream
  // is being captured, not for the small-batch kernel, not from the entry point that must not
  // allocate (an event's first record may), and `fork` = 0 (tuning) switches it off.
  bool forked = false;
  std::unique_lock<std::mutex> fork_lock(tbe->fork_mutex, std::defer_lock);
  if (tbe->side != nullptr && balanced && !one_stream && g_ovr.fork != 0) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone) {
      fork_lock.lock();
      TRA_HIP(hipEventRecord(tbe->ev_fork, s));
      TRA_HIP(hipStreamWaitEvent(tbe->side, tbe->ev_fork, 0));
      forked = true;
    } else {
      (void)hipGetLastError();
    }
  }
  hipStream_t const caller_stream = s;
  // (an error on the way still joins the side streams before it is returned)
  auto join = [&](int rc) -> int {
    if (forked && (hipEventRecord(tbe->ev_join, tbe->side) != hipSuccess ||
                   hipStreamWaitEvent(caller_stream, tbe->ev_join, 0) != hipSuccess)) {
      if (rc == TRA_OK) rc = hip_fail(hipGetLastError(), "joining the second stream of a lookup call");
    }
    return rc;
  };
  for (const int ci : tbe->launch_order) {
    s = forked && tbe->on_side[ci] ? tbe->side : caller_stream;
    const LaunchClass& cls = tbe->classes[ci];
    const ClassGeometry& cg = geo_local.cls[ci];
    LookupArgs a = tbe->base_args[ci];
    a.weights = (const uint8_t*)weights;
    // Lanes past the end of their bag still issue (clamped) id loads, so the
    // kernels need one readable element even when there are no ids at all.
    a.indices = num_indices > 0 ? indices : (const void*)tbe->err_dev;
    a.offsets = offsets;
    // (no ids: nothing to weigh, and the weights pointer may not be readable)
    a.psw = nobag || num_indices == 0 ? nullptr : per_sample_weights;
    if (pw != nullptr && !nobag && num_indices > 0) {
      if (cls.feats.size() > (size_t)kMaxPos) {
        set_error("position-weighted lookup: a launch class has %d features, at most %d are supported",
                  (int)cls.feats.size(), kMaxPos);
        return join(TRA_ERR_TOO_LARGE);
      }
      for (size_t i = 0; i < cls.feats.size(); ++i) {
        const int key = tbe->slices[cls.feats[i]].feature;
        if (key < 0 || key >= pw->num_keys) {
          set_error("position-weighted lookup: feature at key position %d, but %d keys were described", key,
                    pw->num_keys);
          return join(TRA_ERR_INVALID_ARGUMENT);
        }
        const int64_t st = pw->key_start[key], n = pw->key_len[key];
        if (n < 0 || st < 0 || (n > 0 && st + n > pw->table_len)) {
          set_error("position-weighted lookup: key %d has weights [%lld, %lld) outside the table of %lld", key,
                    (long long)st, (long long)(st + n), (long long)pw->table_len);
          return join(TRA_ERR_INVALID_ARGUMENT);
        }
        a.pw_off[i] = (int32_t)st;
        a.pw_len[i] = (int32_t)n;
      }
      a.posw = pw->table;
      a.psw = nullptr;
    }
    a.out = out;
    a.out_stride = out_stride;
    a.bad_to_row0 = tbe->bad_to_row0.load(std::memory_order_relaxed);
    a.num_indices = num_indices > 0 ? num_indices : 1;
    a.B = batch_size;
    a.mean = pooling_mode == TRA_POOL_MEAN;
    a.out_fp16 = out_dtype == TRA_FP16;
    const int ne = cls.cb * 8 / bits_of(cls.dtype);
    bool vec = ((uintptr_t)out % 16 == 0) && ((int64_t)ne * esz % 16 == 0);
    if (nobag) {
      vec = vec && ((int64_t)tbe->dim0 * esz % 16 == 0);
    } else {
      vec = vec && (out_stride * esz % 16 == 0) && (esz == 2 ? cls.cols_aligned_fp16 : cls.cols_aligned_fp32);
    }
    a.vec_store = vec;
    memcpy(a.sub, cg.sub, sizeof(a.sub));
    a.n_sub = cg.n_sub;
    a.xcd_blocks = cg.xcd_blocks;
    a.xcd_count = cg.xcd_count;
    LaunchParams lp;
    lp.balanced = balanced ? 1 : 0;
    lp.lds_bytes = geo_local.tune.lds_bytes;
    lp.grid = cg.grid;
    lp.unroll = geo_local.tune.unroll;
    lp.idx64 = idx_is_i64 != 0;
    lp.weighted = a.psw != nullptr || a.posw != nullptr;
    lp.nobag = nobag;
    lp.from_lengths = from_lengths;
    int rc;
    switch (cls.dtype) {
      case TRA_INT8:
        rc = cls.split ? launch_lookup<TRA_INT8 + kSplitHeader>(a, cls.cb, lp, s) : launch_lookup<TRA_INT8>(a, cls.cb, lp, s);
        break;
      case TRA_INT4:
        rc = cls.split ? launch_lookup<TRA_INT4 + kSplitHeader>(a, cls.cb, lp, s) : launch_lookup<TRA_INT4>(a, cls.cb, lp, s);
        break;
      case TRA_INT2:
        rc = cls.split ? launch_lookup<TRA_INT2 + kSplitHeader>(a, cls.cb, lp, s) : launch_lookup<TRA_INT2>(a, cls.cb, lp, s);
        break;
      case TRA_FP16: rc = launch_lookup<TRA_FP16>(a, cls.cb, lp, s); break;
      default: rc = launch_lookup<TRA_FP32>(a, cls.cb, lp, s); break;
    }
    if (rc != TRA_OK) return join(rc);
  }
  return join(TRA_OK);
}

int tra_tbe_forward(tra_tbe_t tbe, const void* weights, const void* indices,
                    const void* offsets, int32_t idx_is_i64, const float* per_sample_weights,
                    int32_t batch_size, int64_t num_indices, int32_t pooling_mode,
                    int32_t out_dtype, void* out, int64_t out_stride, void* stream) {
  return forward_impl(tbe, weights, indices, offsets, false, idx_is_i64, per_sample_weights,
                      batch_size, num_indices, pooling_mode, out_dtype, out, out_stride, stream);
}

int64_t tra_tbe_forward_lengths_workspace_bytes(int32_t num_keys, int32_t batch_size,
                                                int32_t idx_is_i64) {
  if (num_keys < 0 || batch_size < 0) return 0;
  const int64_t n = (int64_t)num_keys * batch_size;
  const int64_t off_bytes = ((n + 1) * (idx_is_i64 ? 8 : 4) + 255) / 256 * 256;
  return off_bytes + tra_cumsum_workspace_bytes(n);
}

}  // extern "C"

static int forward_lengths_impl(tra_tbe_t tbe, const void* weights, const void* indices,
                                const void* lengths, int32_t idx_is_i64,
                                const float* per_sample_weights, int32_t batch_size,
                                int32_t num_keys, int64_t num_indices, int32_t pooling_mode,
                                int32_t out_dtype, void* out, int64_t out_stride, void* workspace,
                                void* stream, const PositionWeights* pw, bool one_stream = false) {
  if (!tbe) {
    set_error("tra_tbe_forward_lengths: null plan");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (num_keys < 0 || batch_size < 0 || num_indices < 0) {
    set_error("tra_tbe_forward_lengths: negative size");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  for (const FeatureDesc& d : tbe->slices)
    if (d.feature >= num_keys) {
      set_error("tra_tbe_forward_lengths: feature position %d but only %d keys", d.feature,
                num_keys);
      return TRA_ERR_INVALID_ARGUMENT;
    }
  if (!lengths && (int64_t)num_keys * batch_size > 0) {
    set_error("tra_tbe_forward_lengths: null lengths");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (fused_scan_possible(tbe, batch_size, num_keys, num_indices, pooling_mode, lengths) ||
      small_fused_scan_possible(tbe, batch_size, num_keys, num_indices, pooling_mode, lengths))
    return forward_impl(tbe, weights, indices, lengths, true, idx_is_i64, per_sample_weights,
                        batch_size, num_indices, pooling_mode, out_dtype, out, out_stride, stream, pw, one_stream);
  // Offsets first, then the ordinary lookup.
  const int64_t n = (int64_t)num_keys * batch_size;
  if (!workspace) {
    set_error("tra_tbe_forward_lengths: workspace of %lld bytes required",
              (long long)tra_tbe_forward_lengths_workspace_bytes(num_keys, batch_size, idx_is_i64));
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int64_t off_bytes = ((n + 1) * (idx_is_i64 ? 8 : 4) + 255) / 256 * 256;
  void* scan_ws = tra_cumsum_workspace_bytes(n) ? (void*)((uint8_t*)workspace + off_bytes) : nullptr;
  const int rc = tra_cumsum(lengths, n, idx_is_i64, workspace, scan_ws, stream);
  if (rc != TRA_OK) return rc;
  return forward_impl(tbe, weights, indices, workspace, false, idx_is_i64, per_sample_weights,
                      batch_size, num_indices, pooling_mode, out_dtype, out, out_stride, stream, pw, one_stream);
}

extern "C" {

int tra_tbe_forward_lengths(tra_tbe_t tbe, const void* weights, const void* indices,
                            const void* lengths, int32_t idx_is_i64,
                            const float* per_sample_weights, int32_t batch_size, int32_t num_keys,
                            int64_t num_indices, int32_t pooling_mode, int32_t out_dtype, void* out,
                            int64_t out_stride, void* workspace, void* stream) {
  return forward_lengths_impl(tbe, weights, indices, lengths, idx_is_i64, per_sample_weights,
                              batch_size, num_keys, num_indices, pooling_mode, out_dtype, out,
                              out_stride, workspace, stream, nullptr);
}

int64_t tra_tbe_forward_lengths_static_max_bytes(void) { return kStaticScratchBytes; }

int tra_tbe_forward_lengths_static(tra_tbe_t tbe, const void* weights, const void* indices,
                                   const void* lengths, int32_t idx_is_i64,
                                   const float* per_sample_weights, int32_t batch_size,
                                   int32_t num_keys, int64_t num_indices, int32_t pooling_mode,
                                   int32_t out_dtype, void* out, int64_t out_stride, void* stream) {
  if (!tbe) {
    set_error("tra_tbe_forward_lengths_static: null plan");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const int64_t need = tra_tbe_forward_lengths_workspace_bytes(num_keys, batch_size, idx_is_i64);
  if (need > kStaticScratchBytes) {
    set_error("tra_tbe_forward_lengths_static: %d keys x %d samples need %lld bytes of scratch, the static "
              "buffer holds %lld; use tra_tbe_forward_lengths with a workspace",
              num_keys, batch_size, (long long)need, (long long)kStaticScratchBytes);
    return TRA_ERR_TOO_LARGE;
  }
  if (!tbe->static_scratch) {
    set_error("tra_tbe_forward_lengths_static: the static scratch was not resolved for device %d", tbe->device);
    return TRA_ERR_HIP;
  }
  return forward_lengths_impl(tbe, weights, indices, lengths, idx_is_i64, per_sample_weights,
                              batch_size, num_keys, num_indices, pooling_mode, out_dtype, out,
                              out_stride, tbe->static_scratch, stream, nullptr, /*one_stream=*/true);
}

int tra_tbe_forward_position_weighted(tra_tbe_t tbe, const void* weights, const void* indices,
                                      const void* bags, int32_t bags_are_lengths,
                                      int32_t idx_is_i64, const float* position_weights,
                                      int64_t position_weights_len, const int32_t* key_start,
                                      const int32_t* key_len, int32_t num_keys, int32_t batch_size,
                                      int64_t num_indices, int32_t pooling_mode, int32_t out_dtype,
                                      void* out, int64_t out_stride, void* workspace,
                                      void* stream) {
  if (!position_weights || position_weights_len < 1 || !key_start || !key_len || num_keys < 0) {
    set_error("tra_tbe_forward_position_weighted: null or empty position weight description");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (pooling_mode == TRA_POOL_NONE) {
    set_error("tra_tbe_forward_position_weighted: position weights apply to pooled lookups only");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  const PositionWeights pw{position_weights, position_weights_len, key_start, key_len, num_keys};
  if (bags_are_lengths)
    return forward_lengths_impl(tbe, weights, indices, bags, idx_is_i64, nullptr, batch_size,
                                num_keys, num_indices, pooling_mode, out_dtype, out, out_stride,
                                workspace, stream, &pw);
  return forward_impl(tbe, weights, indices, bags, false, idx_is_i64, nullptr, batch_size,
                      num_indices, pooling_mode, out_dtype, out, out_stride, stream, &pw);
}

int tra_tbe_set_bounds_check_mode(tra_tbe_t tbe, int32_t mode) {
  if (!tbe) {
    set_error("tra_tbe_set_bounds_check_mode: null plan");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  if (mode < -1 || mode > 3) {
    set_error("tra_tbe_set_bounds_check_mode: mode %d is none of FATAL 0, WARNING 1, IGNORE 2, NONE 3, unset -1", mode);
    return TRA_ERR_INVALID_ARGUMENT;
  }
  tbe->bad_to_row0.store(mode == 1 || mode == 2 ? 1 : 0, std::memory_order_relaxed);
  return TRA_OK;
}

int tra_tbe_error_count(tra_tbe_t tbe, void* stream, int64_t* count) {
  if (!tbe || !count) {
    set_error("tra_tbe_error_count: null argument");
    return TRA_ERR_INVALID_ARGUMENT;
  }
  unsigned long long v = 0;
  hipStream_t s = (hipStream_t)stream;
  TRA_HIP(hipMemcpyAsync(&v, tbe->err_dev, sizeof(v), hipMemcpyDeviceToHost, s));
  TRA_HIP(hipStreamSynchronize(s));
  if (v != 0) {
    TRA_HIP(hipMemsetAsync(tbe->err_dev, 0, sizeof(v), s));
    TRA_HIP(hipStreamSynchronize(s));
  }
  *count = (int64_t)v;
  return TRA_OK;
}

}  // extern "C"
