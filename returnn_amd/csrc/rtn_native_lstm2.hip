// Host driver and C ABI of the gfx950 NativeLstm2 forward library.
//
// Validates the operator contract (returnn/native_op.py:1054-1068, 1203-1234, 1249-1252), picks a
// decomposition, lays out the caller's workspace and enqueues the kernels of lstm2_kernels.h on the
// caller's stream.  No device memory is allocated here and the stream is never synchronised, so a
// call can sit inside a captured graph like the reference's ops do (returnn/torch/util/graph_capture.py:1-80):
// the persistent kernel is recorded as a kernel node of its own (launch_coresident), per-step modes as their launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>
#include <utility>
#include <vector>

#include <rocblas/rocblas.h>

#include "../../include/rtn_native_lstm2.h"
#include "lstm2_bwd_kernels.h"
#include "lstm2_kernel_tables.h"
#include "lstm2_kernels.h"

// Scratch memory of rtn_native_lstm2_fwd_static, the entry point for callers that cannot allocate: a fixed array in the
// code object, one copy per GPU the library runs on, held until the process ends.  Host code never uses this name as an
// address (on the host it is only a stand-in for the symbol): static_scratch() below asks the runtime for the device
// address once per device and everything else works with that pointer.
#define RTN_STATIC_SCRATCH_BYTES (20u << 20)
static __device__ __align__(256) unsigned char scratch[RTN_STATIC_SCRATCH_BYTES];

namespace rtn {
namespace {

thread_local std::string g_last_error;
thread_local std::string g_plan_text;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

#define RTN_HIP(call)                                                                                  \
  do {                                                                                                 \
    hipError_t err_ = (call);                                                                          \
    if (err_ != hipSuccess)                                                                            \
      return fail(RTN_ERR_HIP, "NativeLstm2: HIP error '%s' in %s (%s:%d)", hipGetErrorString(err_), #call, \
                  __FILE__, __LINE__);                                                                 \
  } while (0)

// The RTN_LSTM2_* environment is read ONCE, into a snapshot (at the first use, and again when the caller asks with
// rtn_native_lstm2_reload_env()): planning does not call getenv per knob and per call, and a setenv in another thread
// cannot race with a reader (readers hold a reference to an immutable snapshot).  `generation` counts the snapshots;
// whatever is cached per plan carries the generation it was made under.
extern "C" char** environ;
struct EnvSnapshot {
  std::unordered_map<std::string, std::string> vars;  // RTN_LSTM2_* only
  unsigned long long generation = 0;
};
std::mutex g_env_mu;
std::shared_ptr<const EnvSnapshot> g_env;
unsigned long long g_env_generation = 0;

std::shared_ptr<const EnvSnapshot> take_env_snapshot() {  // g_env_mu held
  auto snap = std::make_shared<EnvSnapshot>();
  for (char** e = environ; e && *e; ++e) {
    if (strncmp(*e, "RTN_LSTM2_", 10) != 0) continue;
    const char* eq = strchr(*e, '=');
    if (eq) snap->vars.emplace(std::string(*e, eq - *e), std::string(eq + 1));
  }
  snap->generation = ++g_env_generation;
  return snap;
}

std::shared_ptr<const EnvSnapshot> env_snapshot() {
  std::lock_guard<std::mutex> lock(g_env_mu);
  if (!g_env) g_env = take_env_snapshot();
  return g_env;
}

void reload_env() {
  std::lock_guard<std::mutex> lock(g_env_mu);
  g_env = take_env_snapshot();
}

// The value of an RTN_LSTM2_* variable in the snapshot, or nullptr.  (The pointer stays valid while the caller's thread
// holds `keep`, which the accessors below do for the duration of a call through a thread-local reference.)
thread_local std::shared_ptr<const EnvSnapshot> t_env;
const char* env_get(const char* name) {
  t_env = env_snapshot();
  auto it = t_env->vars.find(name);
  return it == t_env->vars.end() ? nullptr : it->second.c_str();
}

long env_long(const char* name, long dflt) {
  const char* v = env_get(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long r = strtol(v, &end, 0);
  return (end && *end == 0) ? r : dflt;
}

struct DeviceInfo {
  int cus = 256;
  int xcds = 8;
  size_t lds_per_wg = 160 * 1024;
  bool cooperative = true;
  bool valid = false;
};

// Properties of the current device; falls back to MI355X's published figures when no device is
// visible (the workspace-size and plan queries must work on a build host without a GPU).
// The XCD count is not among the runtime's device properties.  Until the device has been asked (probe_xcds below, at the
// first call that enqueues work outside stream capture) it is taken to be 8 for devices of 64 CUs or more that divide by
// 8; the kernels check the placement of every group at run time either way.
std::mutex g_dev_mu;
DeviceInfo g_dev_cache[64];
bool g_dev_probed[64] = {false};

DeviceInfo device_info() {
  int dev = 0;
  DeviceInfo fallback;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return fallback;
  }
  // RTN_LSTM2_XCDS: pretend the workgroup ids are dealt to this many XCDs (an experiment and test knob: with a wrong
  // count the groups of an XCD-local plan do not sit on one XCD each, the kernel notices and exchanges at device scope)
  const long env_xcds = env_long("RTN_LSTM2_XCDS", 0);
  std::lock_guard<std::mutex> lock(g_dev_mu);
  if (!g_dev_cache[dev].valid) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      (void)hipGetLastError();
      return fallback;
    }
    DeviceInfo di;
    di.cus = prop.multiProcessorCount;
    di.xcds = (di.cus % 8 == 0 && di.cus >= 64) ? 8 : 1;
    di.lds_per_wg = prop.sharedMemPerBlockOptin ? (size_t)prop.sharedMemPerBlockOptin : (size_t)prop.sharedMemPerBlock;
    if (di.lds_per_wg < (size_t)prop.sharedMemPerBlock) di.lds_per_wg = prop.sharedMemPerBlock;
    di.cooperative = prop.cooperativeLaunch != 0;
    di.valid = true;
    g_dev_cache[dev] = di;
  }
  DeviceInfo di = g_dev_cache[dev];
  if (env_xcds > 0 && di.cus % env_xcds == 0) di.xcds = (int)env_xcds;
  return di;
}

enum PlanKind { kPlanEmpty, kPlanGeneric, kPlanMfma };

struct Plan {
  PlanKind kind = kPlanGeneric;
  int mode = RTN_MODE_STEPWISE;  // resolved: PERSISTENT, GRAPH or STEPWISE
  bool regw = false;             // persistent kernel with W in registers and self-validating exchange
  bool local = false;            // regw: every batch group on one XCD, hidden state exchanged through that XCD's L2
  bool half = false;             // regw: groups of at most 8 rows, two tiles folded into one pass of the pointwise part
  int grid = 0;                  // workgroups launched by the persistent kernel
  int KSMAX = 0;                 // its macro steps per wavefront (template bound)
  int MT = 1, NT = 1;
  int groups = 1, wgs_per_group = 1, Bg = 1, Bp = 16;  // groups: per persistent launch
  int groups_total = 1;          // groups of the whole batch
  int passes = 1;                // persistent launches in turn, each on `groups` of the groups (the last on the rest)
  size_t lds_bytes = 0;
  bool w_direct = false;         // per-step launches read W from memory without an LDS copy
  // workspace layout (byte offsets)
  size_t off_status = 0, off_flags = 0, off_hx = 0, off_wp = 0, off_ycarry = 0, off_trace = 0, total = 0;
  int n_flags = 0;
};

// Most persistent launches in turn that a plan may use instead of the LDS-resident persistent kernel, and instead
// of per-step launches (from step times measured on MI355X).
constexpr int kMaxPassesOverLds = 3;
constexpr int kMaxPassesOverSteps = 12;

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
size_t esize(int dtype) { return dtype == RTN_DTYPE_BF16 ? 2 : 4; }
int round_nt(int nt) { return nt <= 1 ? 1 : (nt <= 2 ? 2 : 4); }

size_t mfma_lds_bytes(int n, int dtype, int MT, int NT) {
  const int KM = dtype == RTN_DTYPE_BF16 ? 32 : 16;
  return (size_t)MT * (n / KM) * kTileBytes + (size_t)kWaves * MT * NT * kTileBytes;
}

// Whether calls made under stream capture keep the persistent kernels (default) or record per-step launches.
bool capture_keeps_persistent() {
  const char* v = env_get("RTN_LSTM2_CAPTURE");
  return !(v && strcmp(v, "steps") == 0);
}

// Chooses the decomposition.  `want_mode` is the caller's mode; `capturing` says the stream is
// under capture (the persistent kernel is then recorded as a graph node, unless RTN_LSTM2_CAPTURE=steps asks for
// per-step launches).  Returns false with a reason when mode == PERSISTENT is impossible.
bool make_plan_uncached(int64_t T, int B, int n, int dtype, int want_mode, bool capturing, Plan* out, std::string* why,
                        int max_wgs_per_cu, int count) {
  Plan pl;
  // One problem on its own is planned with a CU per workgroup (sharing CUs did not pay off in measurements).
  max_wgs_per_cu = (int)std::max<long>(1, std::min<long>(max_wgs_per_cu, env_long("RTN_LSTM2_WGS_PER_CU", 1)));
  const DeviceInfo di = device_info();
  const size_t es = esize(dtype);
  if (T == 0 || B == 0 || n == 0) {
    pl.kind = kPlanEmpty;
    pl.mode = RTN_MODE_STEPWISE;
    pl.total = 256;
    *out = pl;
    return true;
  }
  const bool mfma_shape = (n % 32) == 0;
  const long force_generic = env_long("RTN_LSTM2_FORCE_GENERIC", 0);
  bool persistent_ok = false;
  if (mfma_shape && !force_generic) {
    pl.kind = kPlanMfma;
    // Persistent candidates: every (MT, groups) whose grid fits the device with W on chip.  The register
    // kernel is preferred; among its candidates the estimated step time decides: MFMA cycles of one
    // wavefront plus an exchange term that grows with the number of workgroups that have to hear of
    // each other and with the rows every one of them has to fetch.
    const long env_mt = env_long("RTN_LSTM2_MT", 0);
    const long env_groups = env_long("RTN_LSTM2_GROUPS", 0);
    const long env_kernel = env_long("RTN_LSTM2_KERNEL", 0);  // 0 auto, 1 LDS + flag barrier, 2 registers + self-validating data
    const int KM = dtype == RTN_DTYPE_BF16 ? 32 : 16;
    const int S = n / KM;
    const int ks = (S + kWaves - 1) / kWaves;
    const int KSMAX = ks <= 2 ? 2 : (ks <= 4 ? 4 : (ks <= 8 ? 8 : (ks <= 16 ? 16 : 0)));
    if (want_mode == RTN_MODE_AUTO || want_mode == RTN_MODE_PERSISTENT) {
      struct Cand {
        bool ok = false, regw = false, local = false, half = false;
        int KSMAX = 0, MT = 1, NT = 1, groups = 1, G = 1, Bg = 1, grid = 0;
        size_t lds = 0;
        double est = 1e30;
      };
      // XCD-local decompositions: a group's workgroups (one per CU) all on one XCD, so that the hidden state is handed
      // over through that XCD's L2 (a hand-over between XCDs goes through memory and takes about twice as long).  A group
      // needs G = n / (4 MT) CUs of the XCD; the launch's groups -- those of all `count` problems -- are dealt to the
      // XCDs, floor(CUs per XCD / G) to each.  Fewer rows per group mean fewer bytes for every CU to fetch per step, so
      // the batch is split into as many groups as the device holds.
      auto search_local = [&](int Bq, int problems) {  // Bq rows of each of `problems` problems in one launch
        Cand best;
        const long env_local = env_long("RTN_LSTM2_LOCAL", -1);  // 0: never, 1: whenever feasible, default: by estimate
        if (env_local == 0 || env_kernel == 1 || KSMAX == 0 || di.xcds < 1) return best;
        const int cu_x = di.cus / di.xcds;
        for (int MT : {1, 2, 4, 8}) {
          if (env_mt && MT != env_mt) continue;
          if ((n / 4) % MT) continue;
          const int G = n / (4 * MT);
          // Workgroups that can share a CU: the register kernel with few fragments per wavefront fits twice (two
          // wavefronts per SIMD keep the matrix core busier than one, and one workgroup's MFMAs cover the other's wait).
          const size_t lds_wg = (size_t)regw_lds((int)es, MT, 1).total;
          const int per_cu = (MT * KSMAX <= 32 && KSMAX <= 8 && 2 * lds_wg <= di.lds_per_wg) ? max_wgs_per_cu : 1;
          if (G > cu_x * per_cu) continue;
          if (MT * KSMAX > (KSMAX == 16 ? 32 : 64) || (MT == 8 && KSMAX != 8)) continue;
          const int capacity = di.xcds * (cu_x * per_cu / G) / std::max(problems, 1);  // groups per problem
          if (capacity < 1) continue;
          int groups = std::min(capacity, Bq);
          if (env_groups) groups = (int)std::min<long>(env_groups, groups);
          const int Bg = (Bq + groups - 1) / groups;
          groups = (Bq + Bg - 1) / Bg;
          if ((Bg + 15) / 16 > 4) continue;
          const int NT = round_nt((Bg + 15) / 16);
          if (NT * KSMAX > 32 || MT * NT > 8) continue;
          const bool half = Bg <= 8 && NT == 1 && MT % 2 == 0 && !env_long("RTN_LSTM2_NO_HALF", 0);
          const size_t lds = (size_t)regw_lds((int)es, MT, NT).total;
          if (lds > di.lds_per_wg) continue;
          const double mfma_us = (double)MT * NT * ks * (dtype == RTN_DTYPE_BF16 ? 16 : 128) / 2400.0;
          const int units = half ? MT / 2 : MT * NT;
          const int ept = (units + kWaves - 1) / kWaves;
          // Step time in microseconds, fitted to MI355X measurements (n = 1024 bf16 with 1, 4 and 8 rows per group,
          // n = 512 float32 with 8): a constant, the MFMA issue time of a wavefront and the KB of hidden state every
          // CU fetches per step; a second pass of the pointwise part costs about a quarter of a microsecond.
          const double est = 1.16 + 0.873 * mfma_us + 0.020 * (double)Bg * n * es / 1024.0 + 0.25 * (ept - 1);
          if (est < best.est) {
            best.ok = true; best.regw = true; best.local = true; best.half = half;
            best.est = est; best.KSMAX = KSMAX; best.MT = MT; best.NT = NT; best.groups = groups; best.G = G; best.Bg = Bg;
            best.lds = lds;
            const int total_groups = groups * std::max(problems, 1);
            best.grid = di.xcds * G * ((total_groups + di.xcds - 1) / di.xcds);
          }
        }
        return best;
      };
      // The best persistent decomposition for Bq batch rows in one launch.
      auto search = [&](int Bq, bool regw_only) {
        Cand best;
        for (int use_regw = 1; use_regw >= (regw_only ? 1 : 0); --use_regw) {
          if (use_regw && (env_kernel == 1 || KSMAX == 0)) continue;
          if (!use_regw && (env_kernel == 2 || best.ok)) continue;
          for (int MT : {1, 2, 4, 8}) {
            if (env_mt && MT != env_mt) continue;
            if (MT == 8 && !use_regw) continue;
            if ((n / 4) % MT) continue;
            const int G = n / (4 * MT);
            // Workgroups that can share a CU: the register kernel with few fragments per wavefront fits twice.
            const int per_cu = (use_regw && MT * KSMAX <= 32 && KSMAX <= 8) ? max_wgs_per_cu : 1;
            if (G > di.cus * per_cu) continue;
            if (use_regw && (MT * KSMAX > (KSMAX == 16 ? 32 : 64) || (MT == 8 && KSMAX != 8))) continue;
            const int max_groups = di.cus * per_cu / G;
            for (int groups = 1; groups <= std::min(max_groups, Bq); ++groups) {
              if (env_groups && groups != std::min<long>(env_groups, std::min(max_groups, Bq))) continue;
              const int Bg = (Bq + groups - 1) / groups;
              if ((Bq + Bg - 1) / Bg != groups) continue;  // same rows per group would need fewer groups
              if ((Bg + 15) / 16 > 4) continue;
              const int NT = round_nt((Bg + 15) / 16);
              if (use_regw && (NT * KSMAX > 32 || MT * NT > 8)) continue;  // register budget of one wavefront
              const size_t lds = use_regw ? (size_t)regw_lds((int)es, MT, NT).total : mfma_lds_bytes(n, dtype, MT, NT);
              if (lds > di.lds_per_wg) continue;
              int pc = per_cu;  // workgroups per CU that LDS allows as well
              while (pc > 1 && lds * pc > di.lds_per_wg) --pc;
              if ((long long)groups * G > (long long)di.cus * pc) continue;
              // Step time model fitted to MI355X measurements (microseconds): MFMA issue time of one
              // wavefront, a second round of gate arithmetic when a thread owns two pairs, the number of
              // workgroups that exchange with each other, the fragments a wavefront reads per step and
              // the fragments it holds.
              const double mfma_us = (double)MT * NT * ks * (dtype == RTN_DTYPE_BF16 ? 16 : 128) / 2400.0;
              const int ept = (MT * NT + kWaves - 1) / kWaves;
              double est = 2.0 * mfma_us + 0.4 * (ept - 1) + 0.004 * G + 0.03 * ks * NT + 0.01 * MT * ks;
              // Several problems in one launch: as long as every workgroup has a CU to itself they do not slow
              // each other down; sharing CUs costs about a third, running in turns costs the whole time again.
              if (count > 1) {
                const long long each = (long long)align_up((size_t)(groups * G), (size_t)di.xcds);
                const long long fit1 = di.cus / each, fit2 = 2 * (long long)di.cus / each;
                if (fit1 >= count)
                  ;
                else if (use_regw && fit2 >= count)
                  est *= 1.35;
                else
                  est *= (double)((count + std::max<long long>(fit2, 1) - 1) / std::max<long long>(fit2, 1)) * (fit2 >= 2 ? 1.35 : 1.0);
              }
              if (est < best.est) {
                best.ok = true;
                best.est = est;
                best.regw = use_regw != 0;
                best.KSMAX = use_regw ? KSMAX : 0;
                best.MT = MT;
                best.NT = NT;
                best.groups = groups;
                best.G = G;
                best.Bg = Bg;
                best.lds = lds;
              }
            }
          }
        }
        return best;
      };
      Cand chosen = search(B, false);
      {
        const Cand loc = search_local(B, count);
        // Local or spread?  Measured on MI355X (bf16 n = 192 ... 1024 with 1 ... 128 rows, one and two problems, float32
        // n = 128 ... 512): the hand-over inside an XCD, where all wavefronts of a group wait the same fixed time before
        // their first read, is worth about 0.2 us per step, 0.25 us more once the spread plan keeps more than half of
        // the CUs busy (its exchange then competes for the memory fabric), and 0.005 us for every KB of hidden state
        // that a CU of the spread plan fetches per step beyond what one of the local plan does; against that stands
        // the longer MFMA chain of a wavefront when W is packed into the 32 CUs of one XCD (0.87 us per us of MFMA
        // issue time) and a second pass of the pointwise part (0.25 us).  Problems that would have to share CUs in a
        // spread launch always go local.
        bool take_local = loc.ok && !(chosen.ok && chosen.regw);
        if (loc.ok && chosen.ok && chosen.regw) {
          auto mfma_us = [&](const Cand& c) { return (double)c.MT * c.NT * ks * (dtype == RTN_DTYPE_BF16 ? 16 : 128) / 2400.0; };
          auto passes = [&](const Cand& c) { return ((c.half ? c.MT / 2 : c.MT * c.NT) + kWaves - 1) / kWaves; };
          const long long each = (long long)align_up((size_t)(chosen.groups * chosen.G), (size_t)di.xcds);
          const bool shares = count > 1 && di.cus / each < count;
          const double cost = 0.873 * (mfma_us(loc) - mfma_us(chosen)) + 0.25 * (passes(loc) - passes(chosen));
          const double more_kb = std::max(0, chosen.Bg - loc.Bg) * (double)n * es / 1024.0;  // hidden state per CU and step
          // (bf16: 0.40 since two tiles of a group of up to 8 rows share an accumulator -- measured again at n = 256 ... 1024
          // with 1 ... 64 rows: the XCD-local plan is ahead or level everywhere, a single sequence of n = 1024 included)
          const double gain = (dtype == RTN_DTYPE_BF16 ? 0.40 : 0.20) + (each * std::max(count, 1) > di.cus / 2 ? 0.25 : 0.0) + 0.005 * more_kb;
          take_local = shares || cost < gain;
        }
        if (loc.ok && (env_long("RTN_LSTM2_LOCAL", -1) == 1 || take_local)) chosen = loc;
      }
      // A batch too large for one launch of the register kernel runs as several launches in turn, each on a
      // share of the batch groups (the rows of a batch are independent).  That beats the LDS-resident kernel
      // for a few turns and per-step launches (which read W from HBM every step) for some more.
      if (!(chosen.ok && chosen.regw) && !chosen.local) {
        const long env_passes = env_long("RTN_LSTM2_MAX_PASSES", -1);
        const int limit = (int)(env_passes >= 0 ? env_passes : (chosen.ok ? kMaxPassesOverLds : kMaxPassesOverSteps));
        for (int passes = 2; passes <= std::min(limit, B); ++passes) {
          // (a turn is a launch of one problem; its groups on one XCD each where that is possible: measured at
          // bf16 n = 512 and 1024 with 16 and 32 rows per group, 2.2 us per step and turn against 2.5)
          Cand c = search_local((B + passes - 1) / passes, 1);
          if (!c.ok) c = search((B + passes - 1) / passes, true);
          if (!c.ok) continue;
          if ((((B + c.Bg - 1) / c.Bg) + c.groups - 1) / c.groups > limit) continue;
          chosen = c;
          break;
        }
      }
      if (chosen.ok) {
        pl.regw = chosen.regw;
        pl.local = chosen.local;
        pl.half = chosen.half;
        pl.KSMAX = chosen.KSMAX;
        pl.MT = chosen.MT;
        pl.NT = chosen.NT;
        pl.Bg = chosen.Bg;
        pl.wgs_per_group = chosen.G;
        pl.groups_total = (B + chosen.Bg - 1) / chosen.Bg;
        pl.groups = std::min(chosen.groups, pl.groups_total);
        pl.passes = (pl.groups_total + pl.groups - 1) / pl.groups;
        pl.grid = chosen.local ? chosen.grid : pl.groups * chosen.G;
        pl.lds_bytes = chosen.lds;
        persistent_ok = true;
      }
      if (!persistent_ok && why) *why = "no decomposition keeps W on chip with all workgroups co-resident";
    }
    if (persistent_ok && capturing && !capture_keeps_persistent()) {
      persistent_ok = false;
      if (why) *why = "the stream is being captured and RTN_LSTM2_CAPTURE=steps asks for per-step launches there";
    }
    if (persistent_ok && !di.cooperative) {
      persistent_ok = false;
      if (why) *why = "the device does not support cooperative launches";
    }
    if (!persistent_ok) {
      // Per-step launches have no co-residency limit: 4 cells per workgroup, groups of <= 64 rows.
      int MT = 1;
      pl.regw = false;
      pl.local = pl.half = false;
      pl.KSMAX = 0;
      // A step's launch takes W from memory straight into the matrix cores (every fragment is used once per launch).
      pl.w_direct = env_long("RTN_LSTM2_W_DIRECT", 1) != 0;
      if (!pl.w_direct && mfma_lds_bytes(n, dtype, 1, 4) > di.lds_per_wg) {
        pl.kind = kPlanGeneric;  // copied to LDS first, a W slice of 16 columns does not fit (n far beyond the target sizes)
      } else {
        int groups = (B + 63) / 64;
        int Bg = (B + groups - 1) / groups;
        groups = (B + Bg - 1) / Bg;
        pl.MT = MT;
        pl.NT = round_nt((Bg + 15) / 16);
        pl.groups = pl.groups_total = groups;
        pl.passes = 1;
        pl.wgs_per_group = n / 4;
        pl.Bg = Bg;
        pl.lds_bytes = pl.w_direct ? (size_t)kWaves * pl.MT * pl.NT * kTileBytes : mfma_lds_bytes(n, dtype, pl.MT, pl.NT);
      }
    }
  } else {
    pl.kind = kPlanGeneric;
    if (why) *why = mfma_shape ? "RTN_LSTM2_FORCE_GENERIC is set" : "n is not a multiple of 32";
  }
  if (want_mode == RTN_MODE_PERSISTENT && !persistent_ok) return false;
  if (persistent_ok)
    pl.mode = RTN_MODE_PERSISTENT;
  else if (want_mode == RTN_MODE_STEPWISE || capturing)
    pl.mode = RTN_MODE_STEPWISE;
  else
    pl.mode = RTN_MODE_GRAPH;
  pl.Bp = 16 * pl.NT;

  size_t off = 0;
  pl.off_status = off;
  off += 256;
  pl.off_flags = off;
  pl.n_flags = (pl.kind == kPlanMfma) ? pl.groups_total * pl.wgs_per_group : 0;
  off = align_up(off + (size_t)pl.n_flags * 4, 256);
  if (pl.kind == kPlanMfma) {
    pl.off_hx = off;
    off = align_up(off + (size_t)pl.groups_total * kHxRing * n * pl.Bp * es, 256);
    pl.off_wp = off;
    off = align_up(off + (size_t)4 * n * n * es, 256);
  } else {
    pl.off_ycarry = off;
    off = align_up(off + (size_t)2 * B * n * es, 256);
  }
  if (env_long("RTN_LSTM2_TRACE", 0)) {
    // debugging aid (instrumented builds): 8 cycle totals per workgroup at the end of the workspace
    pl.off_trace = off;
    off = align_up(off + (size_t)1024 * 8 * sizeof(unsigned long long), 256);
  }
  pl.total = off;
  *out = pl;
  return true;
}

// Plans are kept per (shape class, element type, mode, capture state, workgroups per CU, problems per launch, device,
// environment snapshot): the search above runs once per key, and two threads that plan the same call get the same plan.
// (T only matters as "no frames at all".)
struct PlanCacheEntry {
  bool ok;
  Plan plan;
  std::string why;
};
std::mutex g_plan_mu;
std::map<std::tuple<bool, int, int, int, int, bool, int, int, int, unsigned long long>, PlanCacheEntry> g_plans;
constexpr size_t kMaxCachedPlans = 4096;

bool make_plan(int64_t T, int B, int n, int dtype, int want_mode, bool capturing, Plan* out, std::string* why,
               int max_wgs_per_cu = 2, int count = 1) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    dev = -1;
  }
  const auto key = std::make_tuple(T == 0, B, n, dtype, want_mode, capturing, max_wgs_per_cu, count, dev, env_snapshot()->generation);
  {
    std::lock_guard<std::mutex> lock(g_plan_mu);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) {
      if (it->second.ok) *out = it->second.plan;
      if (why) *why = it->second.why;
      return it->second.ok;
    }
  }
  PlanCacheEntry e;
  e.ok = make_plan_uncached(T, B, n, dtype, want_mode, capturing, &e.plan, &e.why, max_wgs_per_cu, count);
  if (e.ok) *out = e.plan;
  if (why) *why = e.why;
  std::lock_guard<std::mutex> lock(g_plan_mu);
  if (g_plans.size() >= kMaxCachedPlans) g_plans.clear();
  g_plans.emplace(key, e);
  return e.ok;
}

void clear_plan_cache() {
  std::lock_guard<std::mutex> lock(g_plan_mu);
  g_plans.clear();
}

const char* mode_name(int mode) {
  switch (mode) {
    case RTN_MODE_PERSISTENT: return "persistent";
    case RTN_MODE_GRAPH: return "graph";
    case RTN_MODE_STEPWISE: return "stepwise";
    default: return "auto";
  }
}

typedef void (*MfmaKernel)(const Lstm2Params, const int, const int);

template <typename AT>
MfmaKernel mfma_kernel_for(int MT, int NT) {
#define RTN_CASE(mt, nt) \
  if (MT == mt && NT == nt) return &k_lstm2_mfma<AT, mt, nt>;
  RTN_CASE(1, 1) RTN_CASE(1, 2) RTN_CASE(1, 4)
  RTN_CASE(2, 1) RTN_CASE(2, 2) RTN_CASE(2, 4)
  RTN_CASE(4, 1) RTN_CASE(4, 2) RTN_CASE(4, 4)
#undef RTN_CASE
  return nullptr;
}

MfmaKernel mfma_kernel(int dtype, int MT, int NT) {
  return dtype == RTN_DTYPE_BF16 ? mfma_kernel_for<__bf16>(MT, NT) : mfma_kernel_for<float>(MT, NT);
}

// Kernels that use more than the default LDS limit need the limit raised once per device.
int ensure_lds_limit(const void* k, size_t lds_bytes) {
  static std::mutex mu;
  static std::list<std::pair<std::pair<int, const void*>, size_t>> done;
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (auto& e : done)
    if (e.first.first == dev && e.first.second == k && e.second >= lds_bytes) return RTN_OK;
  RTN_HIP(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  done.push_back({{dev, k}, lds_bytes});
  return RTN_OK;
}

// Workgroups of a kernel that fit a CU together, asked of the runtime once per (device, kernel, threads, LDS bytes).
int occupancy_per_cu(const void* k, int threads, size_t lds_bytes, int* per_cu) {
  static std::mutex mu;
  static std::map<std::tuple<int, const void*, int, size_t>, int> known;
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  const auto key = std::make_tuple(dev, k, threads, lds_bytes);
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find(key);
    if (it != known.end()) {
      *per_cu = it->second;
      return RTN_OK;
    }
  }
  RTN_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, k, threads, lds_bytes));
  std::lock_guard<std::mutex> lock(mu);
  known[key] = *per_cu;
  return RTN_OK;
}

// Where a sequence of kernel launches goes: onto a stream, or into a graph under construction (one kernel node per launch,
// each depending on the one before).  Every kernel of such a sequence takes the call's parameter block by value as its
// first argument: that is what lets a graph built for one set of buffers be aimed at another set later.
struct GraphNode {
  hipGraphNode_t node = nullptr;
  const void* fn = nullptr;
  dim3 grid, block;
  unsigned lds = 0;
  std::vector<std::vector<char>> args;  // a private copy of every argument
};
struct GraphBuild {
  hipGraph_t graph = nullptr;
  std::vector<GraphNode> nodes;
};
struct LaunchSink {
  hipStream_t stream = nullptr;
  GraphBuild* build = nullptr;  // non-null: add kernel nodes to build->graph instead of launching
};

void node_params(GraphNode& nd, void** ptrs, hipKernelNodeParams* kp) {
  for (size_t i = 0; i < nd.args.size(); ++i) ptrs[i] = nd.args[i].data();
  memset(kp, 0, sizeof(*kp));
  kp->func = const_cast<void*>(nd.fn);
  kp->gridDim = nd.grid;
  kp->blockDim = nd.block;
  kp->sharedMemBytes = nd.lds;
  kp->kernelParams = ptrs;
  kp->extra = nullptr;
}

constexpr size_t kMaxKernelArgs = 8;

template <typename... P, size_t... I>
int enqueue_impl(LaunchSink& sink, void (*k)(P...), dim3 grid, dim3 block, size_t lds, std::tuple<std::decay_t<P>...>& vals,
                 std::index_sequence<I...>) {
  static_assert(sizeof...(P) <= kMaxKernelArgs, "too many kernel arguments");
  void* ptrs[kMaxKernelArgs] = {(void*)&std::get<I>(vals)...};
  if (!sink.build) {
    RTN_HIP(hipLaunchKernel((const void*)k, grid, block, ptrs, lds, sink.stream));
    return RTN_OK;
  }
  GraphNode nd;
  nd.fn = (const void*)k;
  nd.grid = grid;
  nd.block = block;
  nd.lds = (unsigned)lds;
  const size_t sizes[] = {sizeof(std::decay_t<P>)...};
  for (size_t i = 0; i < sizeof...(P); ++i) nd.args.emplace_back((const char*)ptrs[i], (const char*)ptrs[i] + sizes[i]);
  void* own[kMaxKernelArgs];
  hipKernelNodeParams kp;
  node_params(nd, own, &kp);
  std::vector<GraphNode>& nodes = sink.build->nodes;
  hipGraphNode_t before = nodes.empty() ? nullptr : nodes.back().node;
  RTN_HIP(hipGraphAddKernelNode(&nd.node, sink.build->graph, nodes.empty() ? nullptr : &before, nodes.empty() ? 0 : 1, &kp));
  nodes.push_back(std::move(nd));
  return RTN_OK;
}

// Launch k(args...) on the sink's stream, or append it to the sink's graph.
template <typename... P, typename... A>
int enqueue(LaunchSink& sink, void (*k)(P...), dim3 grid, dim3 block, size_t lds, A&&... args) {
  static_assert(sizeof...(P) == sizeof...(A), "argument count does not match the kernel's");
  std::tuple<std::decay_t<P>...> vals(std::forward<A>(args)...);  // converted to the kernel's parameter types
  return enqueue_impl<P...>(sink, k, grid, block, lds, vals, std::index_sequence_for<P...>{});
}

// Library-owned graphs of per-step launch sequences.  The key holds what fixes the structure of the sequence (shape,
// element type, plan, device) and the stream the graph is launched on: no addresses.  A graph whose kernel nodes carry another parameter block than the call's
// (other buffers, same shape) gets the new block written into every node of its executable form before the launch.
struct GraphEntry {
  std::string key;
  std::string block;  // the parameter block the executable graph's nodes carry now
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<GraphNode> nodes;
  hipEvent_t last = nullptr;  // recorded behind every launch: the executable graph may be destroyed once it has completed
};
std::mutex g_graph_mu;
std::list<GraphEntry> g_graphs;   // most recently used first
std::list<GraphEntry> g_retired;  // dropped from g_graphs, possibly still running
constexpr size_t kMaxGraphs = 8;
long long g_graph_records = 0, g_graph_retargets = 0, g_graph_destroyed = 0;

void destroy_entry(GraphEntry& e) {
  if (e.exec) (void)hipGraphExecDestroy(e.exec);
  if (e.graph) (void)hipGraphDestroy(e.graph);
  if (e.last) (void)hipEventDestroy(e.last);
  ++g_graph_destroyed;
}

void sweep_retired() {  // g_graph_mu held
  for (auto it = g_retired.begin(); it != g_retired.end();) {
    if (hipEventQuery(it->last) == hipSuccess) {
      destroy_entry(*it);
      it = g_retired.erase(it);
    } else {
      (void)hipGetLastError();  // hipErrorNotReady is not an error of ours
      ++it;
    }
  }
}

int launch_entry(GraphEntry& e, hipStream_t stream) {
  RTN_HIP(hipGraphLaunch(e.exec, stream));
  RTN_HIP(hipEventRecord(e.last, stream));
  return RTN_OK;
}

template <typename T>
void key_append(std::string* key, const T& v) {
  key->append(reinterpret_cast<const char*>(&v), sizeof(T));
}

// Launches the graph kept for `key` with the parameter block [block, block + bytes) in the first argument of every
// kernel node; builds the graph first (by calling `record` with a sink that collects nodes) if there is none.
// An executable graph is only ever launched on the stream it was first launched on (the stream is part of the key): its
// launches are then ordered by that stream, the one event behind the last of them covers them all when the entry is
// retired, and rewriting its nodes' parameters never meets a launch of the same executable graph running on another stream.
template <typename Record>
int replay_graph(const std::string& shape_key, const void* block, size_t bytes, hipStream_t stream, Record record) {
  std::string key(shape_key);
  key_append(&key, stream);
  std::lock_guard<std::mutex> lock(g_graph_mu);
  sweep_retired();
  for (auto it = g_graphs.begin(); it != g_graphs.end(); ++it) {
    if (it->key != key) continue;
    g_graphs.splice(g_graphs.begin(), g_graphs, it);
    GraphEntry& e = g_graphs.front();
    if (e.block.size() != bytes || memcmp(e.block.data(), block, bytes) != 0) {
      // Other buffers than last time.  Launches of the executable graph that are already queued keep the arguments
      // they were queued with; the update only shows in launches made after it.
      for (GraphNode& nd : e.nodes) {
        memcpy(nd.args[0].data(), block, bytes);
        void* ptrs[kMaxKernelArgs];
        hipKernelNodeParams kp;
        node_params(nd, ptrs, &kp);
        RTN_HIP(hipGraphExecKernelNodeSetParams(e.exec, nd.node, &kp));
      }
      e.block.assign((const char*)block, bytes);
      ++g_graph_retargets;
    }
    return launch_entry(e, stream);
  }
  GraphEntry e;
  e.key = key;
  e.block.assign((const char*)block, bytes);
  GraphBuild build;
  RTN_HIP(hipGraphCreate(&build.graph, 0));
  LaunchSink sink;
  sink.build = &build;
  int rc = record(sink);
  for (GraphNode& nd : build.nodes)
    if (rc == RTN_OK && (nd.args.empty() || nd.args[0].size() != bytes))
      rc = fail(RTN_ERR_HIP, "NativeLstm2: a kernel recorded into a library graph does not take the parameter block first");
  if (rc != RTN_OK) {
    (void)hipGraphDestroy(build.graph);
    return rc;
  }
  e.graph = build.graph;
  e.nodes = std::move(build.nodes);
  hipError_t err = hipGraphInstantiate(&e.exec, e.graph, nullptr, nullptr, 0);
  if (err == hipSuccess) err = hipEventCreateWithFlags(&e.last, hipEventDisableTiming);
  if (err != hipSuccess) {
    destroy_entry(e);
    return fail(RTN_ERR_HIP, "NativeLstm2: building a graph of %zu launches: %s", e.nodes.size(), hipGetErrorString(err));
  }
  ++g_graph_records;
  g_graphs.push_front(std::move(e));
  while (g_graphs.size() > kMaxGraphs) {
    // may still be running on some stream: parked until the event behind its last launch has completed
    g_retired.splice(g_retired.end(), g_graphs, std::prev(g_graphs.end()));
  }
  return launch_entry(g_graphs.front(), stream);
}

int launch_steps(const Lstm2Params& p, const Plan& pl, int dtype, LaunchSink& sink) {
  if (pl.kind == kPlanMfma) {
    MfmaKernel k = mfma_kernel(dtype, pl.MT, pl.NT);
    const dim3 grid(pl.groups * pl.wgs_per_group), block(kWgThreads);
    for (int s = 0; s < p.nsteps; ++s) {
      const int rc = enqueue(sink, k, grid, block, pl.lds_bytes, p, s, s + 1);
      if (rc != RTN_OK) return rc;
    }
  } else {
    const long long bn = (long long)p.B * p.n;
    const dim3 grid((unsigned)((bn + 255) / 256)), block(256);
    for (int s = 0; s < p.nsteps; ++s) {
      const int rc = dtype == RTN_DTYPE_BF16 ? enqueue(sink, k_step_generic<__bf16>, grid, block, 0, p, s)
                                             : enqueue(sink, k_step_generic<float>, grid, block, 0, p, s);
      if (rc != RTN_OK) return rc;
    }
  }
  return RTN_OK;
}

int launch_steps(const Lstm2Params& p, const Plan& pl, int dtype, hipStream_t stream) {
  LaunchSink sink;
  sink.stream = stream;
  return launch_steps(p, pl, dtype, sink);
}

int launch_steps_graph(const Lstm2Params& p, const Plan& pl, int dtype, hipStream_t stream) {
  std::string key("fwd");
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  Lstm2Params shape = p;  // the caller zeroed p before filling it in: padding compares equal
  shape.X = shape.W = shape.y0 = nullptr;
  shape.c0 = shape.mask = nullptr;
  shape.Y = shape.H = nullptr;
  shape.C = shape.d = nullptr;
  shape.status = shape.flags = nullptr;
  shape.hx = shape.Wp = shape.ycarry = nullptr;
  shape.trace = nullptr;
  key.append(reinterpret_cast<const char*>(&shape), sizeof(shape));
  key_append(&key, dtype); key_append(&key, pl.MT); key_append(&key, pl.NT); key_append(&key, (int)pl.kind);
  key_append(&key, pl.lds_bytes); key_append(&key, dev);
  return replay_graph(key, &p, sizeof(p), stream, [&](LaunchSink& sink) { return launch_steps(p, pl, dtype, sink); });
}

// ---- launches that need all their workgroups on the device together ------------------------------------------------
// Outside stream capture: an ordinary launch behind an ordering of the library's own (below).
// Under stream capture a cooperative launch cannot be recorded with the stream API, so the kernel node is built by hand:
// the capturing graph and the stream's current dependencies are asked of the runtime, a kernel node with the cooperative
// attribute is added behind them and made the stream's new dependency.  If the runtime refuses any of that, the kernel
// is recorded as an ordinary kernel node (it never uses a grid barrier; what it needs is co-residency, which the
// occupancy check before the call has established for a device that runs nothing else at that moment; every wait inside
// is bounded, so a replay that does find the device shared ends with the status word set and NaN marks, not hung).
// RTN_LSTM2_CAPTURE_NODE=plain skips the attempt; RTN_LSTM2_CAPTURE=steps records per-step launches as before.
thread_local std::string g_bwd_plan_text;  // what the last gradient call of this thread ran on
std::mutex g_capture_mu;
long long g_capture_cooperative = 0, g_capture_plain = 0;
std::string g_capture_refusal;  // why a cooperative node was refused, if it was

// Outside capture a persistent kernel goes out as an ORDINARY launch.  It uses no grid barrier; what it needs is all its
// workgroups on the device together, which the caller has checked against the occupancy of the kernel, and which an
// ordinary launch gives on a device that is not shared: its waits are bounded like everywhere else.  A cooperative launch
// costs two switches of hardware queue (measured: the device idles 11 us in front of the kernel and 11 us behind it; an
// ordinary launch follows the kernel before it without a gap).  What the cooperative queue did give is that two
// persistent kernels never share the device, each with part of its grid, waiting for the rest: the library keeps that
// property for its own launches itself -- one event per device behind the last persistent launch, which a launch on
// another stream waits for (on the device, the host never blocks).
// RTN_LSTM2_LAUNCH=cooperative brings the cooperative launch back; the entry that may not create anything at call time
// (g_no_setup_objects) keeps it, since this scheme needs an event, and joins the ordering where the event exists.
thread_local bool g_no_setup_objects = false;
struct PersistentOrder {
  hipEvent_t last = nullptr;      // behind the last persistent launch on this device
  hipStream_t stream = nullptr;   // the stream it went to
  bool any = false;
};
std::mutex g_order_mu;
PersistentOrder g_order[64];

int launch_coresident(const void* k, dim3 grid, dim3 block, void** args, unsigned lds, hipStream_t stream, bool capturing) {
  if (!capturing) {
    const char* how = env_get("RTN_LSTM2_LAUNCH");
    int dev = 0;
    RTN_HIP(hipGetDevice(&dev));
    if ((how && strcmp(how, "cooperative") == 0) || dev < 0 || dev >= 64) {
      RTN_HIP(hipLaunchCooperativeKernel(k, grid, block, args, lds, stream));
      return RTN_OK;
    }
    std::lock_guard<std::mutex> lock(g_order_mu);
    PersistentOrder& o = g_order[dev];
    if (g_no_setup_objects) {
      // Cooperative launch, and part of the ordering as far as that takes no new object: behind the last ordinary
      // persistent launch if there has been one on this device, and in front of the next.  (Before the first ordinary
      // launch there is no event to record into: such a call is only ordered by its own stream -- as calls of that entry
      // have to be anyway, since they share one scratch array.)
      if (o.last && o.any && o.stream != stream) RTN_HIP(hipStreamWaitEvent(stream, o.last, 0));
      RTN_HIP(hipLaunchCooperativeKernel(k, grid, block, args, lds, stream));
      if (o.last) {
        RTN_HIP(hipEventRecord(o.last, stream));
        o.stream = stream;
        o.any = true;
      }
      return RTN_OK;
    }
    if (!o.last) RTN_HIP(hipEventCreateWithFlags(&o.last, hipEventDisableTiming));
    if (o.any && o.stream != stream) RTN_HIP(hipStreamWaitEvent(stream, o.last, 0));
    RTN_HIP(hipLaunchKernel(k, grid, block, args, lds, stream));
    RTN_HIP(hipEventRecord(o.last, stream));
    o.stream = stream;
    o.any = true;
    return RTN_OK;
  }
  const char* kind = env_get("RTN_LSTM2_CAPTURE_NODE");
  bool try_cooperative = !(kind && strcmp(kind, "plain") == 0);
  {
    std::lock_guard<std::mutex> lock(g_capture_mu);
    if (!g_capture_refusal.empty()) try_cooperative = false;  // refused once: do not ask again
  }
  if (try_cooperative) {
    hipGraphNode_t node = nullptr;
    const char* step = "hipStreamGetCaptureInfo_v2";
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    hipGraph_t graph = nullptr;
    const hipGraphNode_t* deps = nullptr;
    size_t ndeps = 0;
    hipError_t e = hipStreamGetCaptureInfo_v2(stream, &st, nullptr, &graph, &deps, &ndeps);
    if (e == hipSuccess && (st != hipStreamCaptureStatusActive || !graph)) e = hipErrorIllegalState;
    if (e == hipSuccess) {
      step = "hipGraphAddKernelNode";
      hipKernelNodeParams kp;
      memset(&kp, 0, sizeof(kp));
      kp.func = const_cast<void*>(k);
      kp.gridDim = grid;
      kp.blockDim = block;
      kp.sharedMemBytes = lds;
      kp.kernelParams = args;
      e = hipGraphAddKernelNode(&node, graph, deps, ndeps, &kp);
    }
    if (e == hipSuccess) {
      step = "hipGraphKernelNodeSetAttribute(cooperative)";
      hipKernelNodeAttrValue v;
      memset(&v, 0, sizeof(v));
      v.cooperative = 1;
      e = hipGraphKernelNodeSetAttribute(node, hipKernelNodeAttributeCooperative, &v);
    }
    if (e == hipSuccess) {
      step = "hipStreamUpdateCaptureDependencies";
      e = hipStreamUpdateCaptureDependencies(stream, &node, 1, hipStreamSetCaptureDependencies);
    }
    if (e == hipSuccess) {
      std::lock_guard<std::mutex> lock(g_capture_mu);
      ++g_capture_cooperative;
      return RTN_OK;
    }
    if (node) (void)hipGraphDestroyNode(node);
    (void)hipGetLastError();
    std::lock_guard<std::mutex> lock(g_capture_mu);
    g_capture_refusal = std::string(step) + ": " + hipGetErrorString(e);
  }
  RTN_HIP(hipLaunchKernel(k, grid, block, args, lds, stream));
  std::lock_guard<std::mutex> lock(g_capture_mu);
  ++g_capture_plain;
  return RTN_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_dims(int64_t T, int32_t B, int32_t n, int32_t dtype) {
  if (T < 0 || B < 0 || n < 0) return fail(RTN_ERR_SHAPE, "NativeLstm2: negative dimension (T=%lld, B=%d, n=%d)", (long long)T, B, n);
  if (dtype != RTN_DTYPE_F32 && dtype != RTN_DTYPE_BF16) return fail(RTN_ERR_ARG, "NativeLstm2: unknown dtype %d", dtype);
  if (T > 0x7fffffffLL) return fail(RTN_ERR_SHAPE, "NativeLstm2: T=%lld exceeds the supported 2^31-1 frames", (long long)T);
  if ((long long)B * n > 0x7fffffffLL / 16 || (long long)n * n > 0x7fffffffLL / 16)
    return fail(RTN_ERR_SHAPE, "NativeLstm2: B*n or n*n too large (B=%d, n=%d)", B, n);
  return RTN_OK;
}


// Workspace of one problem of an entry with `count` problems: the largest layout any resolution of `mode`
// can need (AUTO may fall back to per-step launches, and the plan depends on how many problems share a launch).
// ---- widths the matrix-core kernels do not take ------------------------------------------------------------------
// n that is not a multiple of 32 runs zero-padded to the next multiple: a padded cell has zero inputs, zero weights (rows
// and columns) and a zero initial state, so its cell state and output are exactly 0 in every frame, it adds nothing to
// the other cells' sums and all its gradients are 0 -- the results are those of the unpadded problem.  The copies cost
// about the op's own memory traffic again, far less than the element-wise kernels that such widths would otherwise
// run on (n=1000: 120 times slower).  Widths up to 32 stay on those kernels; RTN_LSTM2_NO_PAD=1 switches the padding off.
int padded_width(int n) {
  if (n % 32 == 0 || n <= 32 || env_long("RTN_LSTM2_NO_PAD", 0)) return n;
  return (n + 31) / 32 * 32;
}

// Padded copies of one forward call's tensors (byte offsets into its share of the workspace).
struct FwdPadLayout {
  size_t X = 0, W = 0, y0 = 0, c0 = 0, Y = 0, C = 0, H = 0, d = 0, total = 0;
};
FwdPadLayout fwd_pad_layout(int64_t T, int B, int np, int dtype) {
  const size_t es = esize(dtype), tb = (size_t)T * B, bn = (size_t)B * np;
  FwdPadLayout l;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off = align_up(off + bytes, 256); return at; };
  l.X = take(tb * 4 * np * es);
  l.W = take((size_t)np * 4 * np * es);
  l.y0 = take(bn * es);
  l.c0 = take(bn * 4);
  l.Y = take(tb * np * es);
  l.C = take(tb * np * 4);
  l.H = take(tb * 4 * np * es);
  l.d = take(bn * 4);
  l.total = off;
  return l;
}

// Padded copies of one gradient call's tensors.
struct BwdPadLayout {
  size_t W = 0, y0 = 0, c0 = 0, Y = 0, C = 0, H = 0, DY = 0, Dd = 0, DX = 0, DW = 0, Dy0 = 0, Dc0 = 0, total = 0;
};
BwdPadLayout bwd_pad_layout(int64_t T, int B, int np, int dtype) {
  const size_t es = esize(dtype), tb = (size_t)T * B, bn = (size_t)B * np;
  BwdPadLayout l;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off = align_up(off + bytes, 256); return at; };
  l.W = take((size_t)np * 4 * np * es);
  l.y0 = take(bn * es);
  l.c0 = take(bn * 4);
  l.Y = take(tb * np * es);
  l.C = take(tb * np * 4);
  l.H = take(tb * 4 * np * es);
  l.DY = take(tb * np * es);
  l.Dd = take(bn * 4);
  l.DX = take(tb * 4 * np * es);
  l.DW = take((size_t)np * 4 * np * 4);
  l.Dy0 = take(bn * es);
  l.Dc0 = take(bn * 4);
  l.total = off;
  return l;
}

// dst[rows_dst][blocks][np] := src[rows_src][blocks][n], zeros elsewhere; elements of `es` bytes.
int launch_pad(const void* src, void* dst, long long rows_src, long long rows_dst, int blocks, int n, int np, size_t es, hipStream_t stream,
               long long src_pitch = 0) {
  const long long total = rows_dst * blocks * np;
  if (total <= 0) return RTN_OK;
  if (src_pitch == 0) src_pitch = (long long)blocks * n;
  const dim3 grid((unsigned)std::min<long long>((total + 255) / 256, 8192)), block(256);
  if (es == 2)
    hipLaunchKernelGGL(k_pad_cells<unsigned short>, grid, block, 0, stream, (const unsigned short*)src, (unsigned short*)dst, rows_src, rows_dst, blocks, n, np, src_pitch);
  else
    hipLaunchKernelGGL(k_pad_cells<unsigned>, grid, block, 0, stream, (const unsigned*)src, (unsigned*)dst, rows_src, rows_dst, blocks, n, np, src_pitch);
  RTN_HIP(hipGetLastError());
  return RTN_OK;
}

// dst[rows][blocks][n] := src[rows][blocks][np]; dst_pitch: elements from one row of dst to the next (0: blocks * n).
int launch_unpad(const void* src, void* dst, long long rows, int blocks, int n, int np, size_t es, hipStream_t stream, long long dst_pitch = 0) {
  const long long total = rows * blocks * n;
  if (total <= 0) return RTN_OK;
  if (dst_pitch == 0) dst_pitch = (long long)blocks * n;
  const dim3 grid((unsigned)std::min<long long>((total + 255) / 256, 8192)), block(256);
  if (es == 2)
    hipLaunchKernelGGL(k_unpad_cells<unsigned short>, grid, block, 0, stream, (const unsigned short*)src, (unsigned short*)dst, rows, blocks, n, np, dst_pitch);
  else
    hipLaunchKernelGGL(k_unpad_cells<unsigned>, grid, block, 0, stream, (const unsigned*)src, (unsigned*)dst, rows, blocks, n, np, dst_pitch);
  RTN_HIP(hipGetLastError());
  return RTN_OK;
}

// rows x row_elems elements := 0, rows pitch elements apart (row_elems * es a multiple of 4)
int launch_clear_rows(void* dst, long long rows, long long row_elems, long long pitch, size_t es, hipStream_t stream) {
  if (rows <= 0 || row_elems <= 0) return RTN_OK;
  if (pitch == row_elems) {
    hipLaunchKernelGGL(k_fill_u32, dim3(1024), dim3(256), 0, stream, (unsigned*)dst, 0u, (long long)((size_t)rows * row_elems * es / 4));
  } else {
    hipLaunchKernelGGL(k_clear_rows, dim3(1024), dim3(256), 0, stream, (unsigned*)dst, rows, (long long)((size_t)row_elems * es / 4),
                       (long long)((size_t)pitch * es / 4));
  }
  RTN_HIP(hipGetLastError());
  return RTN_OK;
}

// Row pitch of a call's array: what the caller gave, or the contiguous one; checked against what the kernels assume
// (rows do not overlap, stay 16-byte aligned, and a frame stays within the 32-bit offsets of a buffer descriptor).
int resolve_pitch(const char* name, long long given, long long contiguous, int B, size_t es, long long* out) {
  const long long ld = given ? given : contiguous;
  if (ld < contiguous) return fail(RTN_ERR_ARG, "NativeLstm2: row pitch %s=%lld is below the row length %lld", name, ld, contiguous);
  if (ld != contiguous && ((size_t)ld * es) % 4 != 0) return fail(RTN_ERR_ARG, "NativeLstm2: row pitch %s=%lld must keep rows 4-byte aligned", name, ld);
  // (widths whose contiguous rows are not 16-byte aligned run on element-wise kernels or on padded copies)
  if (((size_t)contiguous * es) % 16 == 0 && ((size_t)ld * es) % 16 != 0)
    return fail(RTN_ERR_ARG, "NativeLstm2: row pitch %s=%lld must keep rows 16-byte aligned", name, ld);
  if ((unsigned long long)B * (unsigned long long)ld * es >= 0xFFFFFF00ull)
    return fail(RTN_ERR_SHAPE, "NativeLstm2: a frame of %d rows with pitch %s=%lld exceeds 4 GiB", B, name, ld);
  *out = ld;
  return RTN_OK;
}

// Workspace of one of `count` forward calls at a width the kernels take as it is.
size_t workspace_each_exact(int count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  size_t need = 0;
  Plan pl;
  std::string why;
  for (int c : {1, std::max(1, std::min(count, kMaxMulti))}) {
    if (make_plan(T, B, n, dtype, mode, false, &pl, &why, 2, c)) need = std::max(need, pl.total);
    if (mode == RTN_MODE_AUTO || mode == RTN_MODE_PERSISTENT) {
      // what the call may settle on when the device gives the kernel fewer workgroups per CU, or none at all
      if (make_plan(T, B, n, dtype, mode, false, &pl, &why, 1, c)) need = std::max(need, pl.total);
      if (make_plan(T, B, n, dtype, RTN_MODE_STEPWISE, true, &pl, &why)) need = std::max(need, pl.total);
    }
  }
  return need;
}

// Workspace of one of `count` forward calls (call k's slice starts at k times this, with its status block first): for a
// padded width, that of the padded problem followed by the padded copies.
size_t workspace_each(int count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  const int np = padded_width(n);
  if (np == n || T == 0 || B == 0) return workspace_each_exact(count, T, B, n, dtype, mode);
  return workspace_each_exact(count, T, B, np, dtype, mode) + fwd_pad_layout(T, B, np, dtype).total;
}

int static_scratch(void** out);
void clear_plan_cache();

// Asks the device once how many XCDs it deals workgroups to: a grid of 1024 small workgroups notes the XCD each runs on
// (hardware register XCC_ID) in a word of the library's static device array, the word comes back over the caller's stream,
// which is waited for -- the one time the library synchronises a stream, at the first call on a device that enqueues
// work outside stream capture.  If the count differs from the assumed one, plans made so far are dropped.
int probe_xcds(hipStream_t stream) {
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return RTN_OK;
  (void)device_info();  // fills the cache entry
  {
    std::lock_guard<std::mutex> lock(g_dev_mu);
    if (g_dev_probed[dev] || !g_dev_cache[dev].valid) return RTN_OK;
    g_dev_probed[dev] = true;  // one attempt
  }
  void* word = nullptr;
  int rc = static_scratch(&word);
  if (rc != RTN_OK) return rc;
  unsigned mask = 0;
  hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, stream, (unsigned*)word, 0u, 64LL);
  hipLaunchKernelGGL(k_probe_xcds, dim3(1024), dim3(64), 0, stream, (unsigned*)word);
  RTN_HIP(hipGetLastError());
  RTN_HIP(hipMemcpyAsync(&mask, word, sizeof(mask), hipMemcpyDeviceToHost, stream));
  RTN_HIP(hipStreamSynchronize(stream));
  int count = 0;
  for (unsigned m = mask; m; m &= m - 1) ++count;
  bool changed = false;
  {
    std::lock_guard<std::mutex> lock(g_dev_mu);
    DeviceInfo& di = g_dev_cache[dev];
    if (count >= 1 && di.cus % count == 0 && di.xcds != count) {
      di.xcds = count;
      changed = true;
    }
  }
  if (changed) clear_plan_cache();
  return RTN_OK;
}

int fwd_calls(const rtn_lstm2_call* calls, int count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode,
              void* workspace, size_t workspace_bytes, void* hip_stream, int op_flags = 0, size_t ws_stride = 0,
              bool no_graph = false);

// The problems zero-padded to a width the matrix-core kernels take (see padded_width), on copies in the workspace: slice
// k = the workspace of the padded call k, then its padded copies.
int fwd_padded(const rtn_lstm2_call* calls, int count, int64_t T, int32_t B, int32_t n, int np, int32_t dtype, int32_t mode,
               void* workspace, size_t workspace_bytes, hipStream_t stream, int op_flags, bool no_graph) {
  int rc = RTN_OK;
  for (int k = 0; k < count; ++k) {
    const rtn_lstm2_call& c = calls[k];
    const void* ptrs[] = {c.X, c.W, c.y0, c.c0, c.i, c.Y, c.C, c.H, c.d};
    const char* names[] = {"X", "W", "y0", "c0", "i", "Y", "C", "H", "d"};
    for (int q = 0; q < 9; ++q)
      if (!ptrs[q]) return fail(RTN_ERR_ARG, "NativeLstm2: %s must not be null", names[q]);
  }
  const size_t inner_each = workspace_each_exact(count, T, B, np, dtype, mode);
  const FwdPadLayout L = fwd_pad_layout(T, B, np, dtype);
  const size_t each = inner_each + L.total;
  const size_t need = (size_t)count * each;
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "NativeLstm2: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "NativeLstm2: workspace must be 16-byte aligned");
  const size_t es = esize(dtype);
  const long long tb = (long long)T * B;
  std::vector<rtn_lstm2_call> padded((size_t)count);
  for (int k = 0; k < count; ++k) {
    const rtn_lstm2_call& c = calls[k];
    unsigned char* base = (unsigned char*)workspace + (size_t)k * each + inner_each;
    long long ldX = 0, ldY = 0;
    if ((rc = resolve_pitch("ldX", c.ldX, 4LL * n, B, es, &ldX)) != RTN_OK) return rc;
    if ((rc = resolve_pitch("ldY", c.ldY, n, B, es, &ldY)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.X, base + L.X, tb, tb, 4, n, np, es, stream, ldX)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.W, base + L.W, n, np, 4, n, np, es, stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.y0, base + L.y0, B, B, 1, n, np, es, stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.c0, base + L.c0, B, B, 1, n, np, 4, stream)) != RTN_OK) return rc;
    padded[(size_t)k] = {base + L.X, base + L.W, base + L.y0, (const float*)(base + L.c0), c.i, c.start, c.step,
                         base + L.Y, (float*)(base + L.C), base + L.H, (float*)(base + L.d), 0, 0};
  }
  rc = fwd_calls(padded.data(), count, T, B, np, dtype, mode, workspace, need, (void*)stream, op_flags, each, no_graph);
  if (rc != RTN_OK) return rc;
  for (int k = 0; k < count; ++k) {
    const rtn_lstm2_call& c = calls[k];
    const rtn_lstm2_call& q = padded[(size_t)k];
    if ((rc = launch_unpad(q.Y, c.Y, tb, 1, n, np, es, stream, c.ldY)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.C, c.C, tb, 1, n, np, 4, stream)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.H, c.H, tb, 4, n, np, es, stream)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.d, c.d, B, 1, n, np, 4, stream)) != RTN_OK) return rc;
  }
  return RTN_OK;
}

// The plan of an entry, settled against the device: a persistent plan needs all its workgroups on the device together,
// so it is checked against what the kernel really gets per CU, planned again for that if it was too optimistic, and
// given up for per-step launches if that does not help.  *pk: the persistent kernel (null: launches per step);
// *fused: problems per persistent launch.
int settle_fwd_plan(int count, int64_t T, int B, int n, int dtype, int mode, bool capturing, Plan* plan, const void** pk, int* fused) {
  Plan& pl = *plan;
  std::string why;
  int rc = RTN_OK;
  *pk = nullptr;
  *fused = 1;
  const int plan_count = env_long("RTN_LSTM2_NO_FUSE", 0) ? 1 : std::min(count, kMaxMulti);
  if (!make_plan(T, B, n, dtype, mode, capturing, &pl, &why, 2, plan_count))
    return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: persistent mode unavailable for T=%lld B=%d n=%d: %s", (long long)T, B, n, why.c_str());
  for (int attempt = 0; pl.kind == kPlanMfma && pl.mode == RTN_MODE_PERSISTENT; ++attempt) {
    *pk = pl.regw ? (const void*)regw_kernel(dtype, pl.MT, pl.NT, pl.KSMAX, pl.half) : (const void*)mfma_kernel(dtype, pl.MT, pl.NT);
    if (!*pk) return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: no kernel for mt=%d nt=%d ks=%d", pl.MT, pl.NT, pl.KSMAX);
    if ((rc = ensure_lds_limit(*pk, pl.lds_bytes)) != RTN_OK) return rc;
    const int wgs = pl.regw ? pl.grid : pl.groups * pl.wgs_per_group;
    int per_cu = 0;
    if ((rc = occupancy_per_cu(*pk, kWgThreads, pl.lds_bytes, &per_cu)) != RTN_OK) return rc;
    const long long capacity = (long long)per_cu * device_info().cus;
    if (capacity >= wgs) {
      if (pl.local) {
        *fused = plan_count;  // the plan's grid holds the groups of that many problems
      } else if (pl.regw && count > 1 && pl.passes == 1 && !env_long("RTN_LSTM2_NO_FUSE", 0)) {
        const long long each = (long long)align_up((size_t)wgs, (size_t)device_info().xcds);
        *fused = (int)std::max<long long>(1, std::min<long long>(std::min(count, kMaxMulti), capacity / each));
      }
      return RTN_OK;
    }
    *pk = nullptr;
    if (attempt == 0 && per_cu >= 1 && make_plan(T, B, n, dtype, mode, capturing, &pl, &why, per_cu, plan_count)) continue;
    if (mode == RTN_MODE_PERSISTENT)
      return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: %d workgroups cannot be co-resident (%d per CU)", wgs, per_cu);
    if (!make_plan(T, B, n, dtype, RTN_MODE_GRAPH, capturing, &pl, &why))
      return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: no per-step plan: %s", why.c_str());
    break;
  }
  return RTN_OK;
}

// The parameter block of call `c` on plan `pl` with its workspace slice at `ws`.
int fill_fwd_params(const rtn_lstm2_call& c, const Plan& pl, bool persistent, unsigned char* ws, int64_t T, int B, int n, int dtype,
                    int op_flags, Lstm2Params* out) {
  Lstm2Params& p = *out;
  int rc = RTN_OK;
  memset(&p, 0, sizeof(p));
  p.X = c.X; p.W = c.W; p.y0 = c.y0; p.c0 = c.c0; p.mask = c.i;
  p.Y = c.Y; p.C = c.C; p.H = c.H; p.d = c.d;
  p.status = (unsigned*)(ws + pl.off_status);
  p.flags = (unsigned*)(ws + pl.off_flags);
  p.hx = ws + pl.off_hx;
  p.Wp = ws + pl.off_wp;
  p.ycarry = ws + pl.off_ycarry;
  p.trace = pl.off_trace ? (unsigned long long*)(ws + pl.off_trace) : nullptr;
  p.T = T; p.B = B; p.n = n;
  if ((rc = resolve_pitch("ldX", c.ldX, 4LL * n, B, esize(dtype), &p.ldX)) != RTN_OK) return rc;
  if ((rc = resolve_pitch("ldY", c.ldY, n, B, esize(dtype), &p.ldY)) != RTN_OK) return rc;
  // returnn/native_op.py:1253-1259
  if (c.step > 0) {
    p.first = c.start;
    p.nsteps = (int)((T - 1 - c.start) / c.step + 1);
  } else {
    p.first = (int)(T - c.start - 1);
    const long long last = (op_flags & kOpEndAtStart) ? c.start : 0;
    if (p.first < last) return fail(RTN_ERR_RANGE, "LstmLowMem: start=%d with a negative step visits no frame of T=%lld", c.start, (long long)T);
    p.nsteps = (int)((p.first - last) / (-(long long)c.step) + 1);
  }
  p.step = c.step;
  p.groups = p.groups_total = pl.groups_total; p.wgs_per_group = pl.wgs_per_group; p.Bg = pl.Bg; p.Bp = pl.Bp;
  p.group_offset = 0;
  p.op_flags = op_flags;
  p.w_direct = (!persistent && pl.kind == kPlanMfma && pl.w_direct) ? 1 : 0;
  p.hx_bufs = kHxRing;
  p.hx_sentinel = pl.regw ? 1 : 0;
  p.exchange = (int)env_long("RTN_LSTM2_EXCHANGE", 0);
  if (p.exchange != kExNoWait) p.exchange = kExDevice;  // no-wait: a timing aid, results invalid (status 2)
  // Device-scope stores take about a microsecond to become visible: a first read issued at once would
  // come back incomplete and cost a second round trip, so it is held back, and the kernel adapts the delay.  Within an
  // XCD the delay is a fixed one (tuned on MI355X over n = 64 ... 1024 and 1 ... 16 rows per group: the best fixed
  // delay is within 2 % of these four everywhere, and 4 % to 13 % ahead of the adaptive one).
  p.poll_delay = (int)std::max<long>(0, std::min<long>(64, env_long("RTN_LSTM2_POLL_DELAY", pl.local ? (pl.Bg > 8 ? 10 : (dtype != RTN_DTYPE_BF16 ? 5 : (pl.MT >= 8 ? 6 : 3))) : 20)));
  {
    long dec = env_long("RTN_LSTM2_DELAY_DEC", 8);  // steps per unit of downward adaptation: a power of two
    int mask = 0;
    while (2 * (mask + 1) <= dec && mask < 255) mask = 2 * mask + 1;
    p.delay_dec_mask = mask;
    p.delay_inc = (int)std::max<long>(0, std::min<long>(16, env_long("RTN_LSTM2_DELAY_INC", pl.local ? 0 : 2)));
  }
  p.xcds = device_info().xcds;
  p.sync_policy = (int)env_long("RTN_LSTM2_SYNC", kStoreCoherent | kLoadCoherent);
  if (!((p.sync_policy & (kStoreCoherent | kReleaseFence)) && (p.sync_policy & (kLoadCoherent | kAcquireFence))))
    return fail(RTN_ERR_ARG, "NativeLstm2: RTN_LSTM2_SYNC=%d is not a valid publication policy", p.sync_policy);
  p.timeout_ticks = (unsigned long long)env_long("RTN_LSTM2_TIMEOUT_TICKS", 200000000L);  // 2 s at 100 MHz
  return RTN_OK;
}

// The calls of one entry: `count` independent problems of one shape.  Each gets the slice
// [k * each, (k + 1) * each) of the workspace, each = workspace_each(count, ...).
// When the persistent register kernel fits that many times on the device at once, all of them run
// in one launch (every workgroup with a CU to itself); otherwise they are enqueued one after the other.
int fwd_calls(const rtn_lstm2_call* calls, int count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode,
              void* workspace, size_t workspace_bytes, void* hip_stream, int op_flags, size_t ws_stride, bool no_graph) {
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (mode < RTN_MODE_AUTO || mode > RTN_MODE_STEPWISE) return fail(RTN_ERR_ARG, "NativeLstm2: unknown mode %d", mode);
  hipStream_t stream = (hipStream_t)hip_stream;
  const long long bn = (long long)B * n;

  for (int k = 0; k < count; ++k)
    if (bn > 0 && (!calls[k].c0 || !calls[k].d)) return fail(RTN_ERR_ARG, "NativeLstm2: c0 and d must not be null");
  if (T == 0 || bn == 0) {
    // returnn/native_op.py:1236-1237: no frames, the final cell state is the initial one.
    for (int k = 0; k < count && bn > 0; ++k) {
      hipLaunchKernelGGL(k_copy_f32, dim3((unsigned)std::min<long long>((bn + 255) / 256, 1024)), dim3(256), 0, stream,
                         calls[k].c0, calls[k].d, bn);
      RTN_HIP(hipGetLastError());
    }
    return RTN_OK;
  }
  const int np = padded_width(n);
  if (np != n) return fwd_padded(calls, count, T, B, n, np, dtype, mode, workspace, workspace_bytes, stream, op_flags, no_graph);
  for (int k = 0; k < count; ++k) {
    const rtn_lstm2_call& c = calls[k];
    if (c.start < 0 || c.start >= T)
      return fail(RTN_ERR_RANGE, "NativeLstm2: need 0 <= start < T, got start=%d, T=%lld", c.start, (long long)T);
    if (c.step == 0) return fail(RTN_ERR_RANGE, "NativeLstm2: step must not be 0");
    const void* ptrs[] = {c.X, c.W, c.y0, c.c0, c.i, c.Y, c.C, c.H, c.d};
    const char* names[] = {"X", "W", "y0", "c0", "i", "Y", "C", "H", "d"};
    for (int q = 0; q < 9; ++q) {
      if (!ptrs[q]) return fail(RTN_ERR_ARG, "NativeLstm2: %s must not be null", names[q]);
      // W is read in 16-byte fragments by the MFMA kernels only (n a multiple of 32); the generic kernels read single
      // elements, which lets LstmLowMem pass the recurrent rows of its stacked matrix at any element offset
      if (q != 4 && !(q == 1 && n % 32 != 0) && !aligned16(ptrs[q]))
        return fail(RTN_ERR_ARG, "NativeLstm2: %s must be 16-byte aligned", names[q]);
    }
  }

  hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
  if (stream) RTN_HIP(hipStreamIsCapturing(stream, &cap_status));
  const bool capturing = cap_status != hipStreamCaptureStatusNone;

  Plan pl;
  const void* pk = nullptr;  // the persistent kernel, if any
  int fused = 1;             // problems per persistent launch
  if ((rc = settle_fwd_plan(count, T, B, n, dtype, mode, capturing, &pl, &pk, &fused)) != RTN_OK) return rc;
  // distance between the calls' workspaces: given by a caller that keeps more than the workspace in a call's slice
  const size_t each_ws = ws_stride ? ws_stride : (count > 1 ? workspace_each(count, T, B, n, dtype, mode) : pl.total);
  if (each_ws < pl.total) return fail(RTN_ERR_WORKSPACE, "NativeLstm2: internal: workspace slice %zu < layout %zu", each_ws, pl.total);
  if (!workspace || workspace_bytes < each_ws * (size_t)count)
    return fail(RTN_ERR_WORKSPACE, "NativeLstm2: workspace of %zu bytes needed, got %zu", each_ws * (size_t)count,
                workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "NativeLstm2: workspace must be 16-byte aligned");
  // (all arguments are in order: from here on work is enqueued.  The first such call on a device asks it for its XCD
  // count; the plan above was made with the assumed count, which the kernels verify for every group anyway.)
  if (!capturing && (rc = probe_xcds(stream)) != RTN_OK) return rc;

  Lstm2Multi multi;
  memset(&multi, 0, sizeof(multi));
  int pending = 0;  // problems prepared for the next persistent launch
  for (int k = 0; k < count; ++k) {
    Lstm2Params p;
    if ((rc = fill_fwd_params(calls[k], pl, pk != nullptr, (unsigned char*)workspace + (size_t)k * each_ws, T, B, n, dtype, op_flags, &p)) != RTN_OK)
      return rc;

    // Frames the loop never visits.
    if (p.nsteps != T) {
      const long long total = T * bn * 4;
      const dim3 grid((unsigned)std::min<long long>((total + 255) / 256, 65535)), block(256);
      if (dtype == RTN_DTYPE_BF16)
        hipLaunchKernelGGL(k_fill_unvisited<__bf16>, grid, block, 0, stream, p);
      else
        hipLaunchKernelGGL(k_fill_unvisited<float>, grid, block, 0, stream, p);
      RTN_HIP(hipGetLastError());
    }

    if (pl.kind == kPlanMfma) {
      MfmaKernel mk = mfma_kernel(dtype, pl.MT, pl.NT);
      if (!pk) {
        if (!mk) return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: no kernel for mt=%d nt=%d", pl.MT, pl.NT);
        rc = ensure_lds_limit((const void*)mk, pl.lds_bytes);
        if (rc != RTN_OK) return rc;
      }
      const long long work = std::max<long long>((long long)n * n, bn);
      const dim3 pgrid((unsigned)std::min<long long>((work + 255) / 256, 2048)), pblock(256);
      // (the problems of a fused launch are prepared by one launch, in front of it)
      const bool prepared_with_the_others = pk && pl.regw && pl.passes <= 1;
      if (!prepared_with_the_others) {
        if (dtype == RTN_DTYPE_BF16)
          hipLaunchKernelGGL(k_prepare_mfma<__bf16>, pgrid, pblock, 0, stream, p, pl.n_flags);
        else
          hipLaunchKernelGGL(k_prepare_mfma<float>, pgrid, pblock, 0, stream, p, pl.n_flags);
        RTN_HIP(hipGetLastError());
      }
      if (pk && pl.regw && pl.passes > 1) {
        // the batch groups in turns: one persistent launch per share of them
        for (int g0 = 0; g0 < pl.groups_total; g0 += pl.groups) {
          Lstm2Multi one;
          memset(&one, 0, sizeof(one));
          one.p[0] = p;
          one.p[0].group_offset = g0;
          one.p[0].groups = std::min(pl.groups, pl.groups_total - g0);
          one.count = 1;
          one.local = pl.local ? 1 : 0;
          one.xcds = device_info().xcds;
          // (an XCD-local turn: the groups dealt to the XCDs, workgroup id = slot * xcds + xcd)
          one.grid = pl.local ? one.xcds * pl.wgs_per_group * ((one.p[0].groups + one.xcds - 1) / one.xcds) : one.p[0].groups * pl.wgs_per_group;
          one.wgs_each = (int)align_up((size_t)one.grid, (size_t)device_info().xcds);
          void* args[] = {(void*)&one};
          rc = launch_coresident(pk, dim3(one.grid), dim3(kWgThreads), args, (unsigned)pl.lds_bytes, stream, capturing);
          if (rc != RTN_OK) return rc;
        }
        continue;
      }
      if (pk && pl.regw) {
        p.groups = pl.groups;
        multi.p[pending++] = p;
        if (pending == fused || k + 1 == count) {
          multi.count = pending;
          multi.grid = pl.grid;
          multi.wgs_each = (int)align_up((size_t)pl.grid, (size_t)device_info().xcds);
          multi.local = pl.local ? 1 : 0;
          multi.xcds = device_info().xcds;
          if (dtype == RTN_DTYPE_BF16)
            hipLaunchKernelGGL(k_prepare_mfma_multi<__bf16>, dim3(pgrid.x, (unsigned)pending), pblock, 0, stream, multi, pl.n_flags);
          else
            hipLaunchKernelGGL(k_prepare_mfma_multi<float>, dim3(pgrid.x, (unsigned)pending), pblock, 0, stream, multi, pl.n_flags);
          RTN_HIP(hipGetLastError());
          void* args[] = {(void*)&multi};
          const int wgs = (pending == 1 || pl.local) ? pl.grid : multi.wgs_each * pending;
          rc = launch_coresident(pk, dim3(wgs), dim3(kWgThreads), args, (unsigned)pl.lds_bytes, stream, capturing);
          if (rc != RTN_OK) return rc;
          pending = 0;
        }
        continue;
      }
      if (pk) {
        p.groups = pl.groups;
        int s_begin = 0, s_end = p.nsteps;
        void* args_lds[] = {(void*)&p, (void*)&s_begin, (void*)&s_end};
        rc = launch_coresident(pk, dim3(pl.groups * pl.wgs_per_group), dim3(kWgThreads), args_lds, (unsigned)pl.lds_bytes, stream, capturing);
        if (rc != RTN_OK) return rc;
        continue;
      }
    } else {
      hipLaunchKernelGGL(k_clear_status, dim3(1), dim3(64), 0, stream, p.status);
      RTN_HIP(hipGetLastError());
    }
    // (a library-owned graph needs a stream, a graph and an executable graph of its own: not for callers that cannot allocate)
    rc = (pl.mode == RTN_MODE_GRAPH && !capturing && !no_graph) ? launch_steps_graph(p, pl, dtype, stream) : launch_steps(p, pl, dtype, stream);
    if (rc != RTN_OK) return rc;
  }
  return RTN_OK;
}


// Bytes of dynamic shared memory of the gradient kernel's variants that keep half of a wavefront's share of W in LDS (4
// wavefronts with 32 + 32 fragments, or 8 wavefronts with 16 + 16).
constexpr size_t kBwdLdsShareBytes = (size_t)kWaves * 32 * 64 * 16;

// One rocBLAS handle per host thread and device, created on first use and kept for the life of the thread (never
// destroyed: at thread or process exit the runtime below it may already be gone).  A handle carries the stream its
// calls go to; with a handle of its own a thread cannot have that stream changed under it by another thread's call.
int blas_handle(rocblas_handle* out) {
  static thread_local rocblas_handle handles[64] = {nullptr};
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(RTN_ERR_HIP, "NativeLstm2: device index %d out of range", dev);
  if (!handles[dev]) {
    if (rocblas_create_handle(&handles[dev]) != rocblas_status_success) {
      handles[dev] = nullptr;
      return fail(RTN_ERR_HIP, "NativeLstm2: rocblas_create_handle failed");
    }
  }
  *out = handles[dev];
  return RTN_OK;
}

// DW[n,4n] (row major, float32) += A[rows,n]^T * Bm[rows,4n] with A, Bm of element type `dtype`, row major.
int dw_accumulate(rocblas_handle h, const void* A, const void* Bm, float* DW, long long rows, int n, int dtype, long long lda = 0,
                  long long ldb = 0) {
  if (rows <= 0) return RTN_OK;
  if (lda == 0) lda = n;
  if (ldb == 0) ldb = 4LL * n;
  const float alpha = 1.f, beta = 1.f;
  const rocblas_datatype in = dtype == RTN_DTYPE_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f32_r;
  // Row-major DW[n,4n] is column-major [4n,n]: DW^T = Bm^T * A, with row-major Bm[rows,4n] = column-major [4n,rows]
  // (no transpose) and row-major A[rows,n] = column-major [n,rows] (transpose).  lda, ldb: row pitch of A and Bm in
  // elements (0: contiguous).
  const rocblas_status st = rocblas_gemm_ex(h, rocblas_operation_none, rocblas_operation_transpose, 4 * n, n, (rocblas_int)rows,
                                            &alpha, Bm, in, (rocblas_int)ldb, A, in, (rocblas_int)lda, &beta, DW, rocblas_datatype_f32_r, 4 * n, DW,
                                            rocblas_datatype_f32_r, 4 * n, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
  if (st != rocblas_status_success) return fail(RTN_ERR_HIP, "NativeLstm2: rocblas_gemm_ex failed with status %d", (int)st);
  return RTN_OK;
}

// Row-major C[M,N] = op(A) * op(B) + beta * C with float32 accumulation.  A is [M,K] (or [K,M] with trans_a), B is [K,N]
// (or [N,K] with trans_b); A and B of element type `in`, C of element type `out`.
int gemm_row_major(rocblas_handle h, bool trans_a, bool trans_b, long long M, long long N, long long K, const void* A, long long lda,
                   const void* Bm, long long ldb, rocblas_datatype in, float beta, void* C, long long ldc, rocblas_datatype out) {
  if (M <= 0 || N <= 0) return RTN_OK;
  const float alpha = 1.f;
  // in column-major terms: C^T [N,M] = op(B)^T * op(A)^T, and a row-major matrix is its transpose in column-major order
  const rocblas_status st = rocblas_gemm_ex(h, trans_b ? rocblas_operation_transpose : rocblas_operation_none,
                                            trans_a ? rocblas_operation_transpose : rocblas_operation_none, (rocblas_int)N, (rocblas_int)M,
                                            (rocblas_int)K, &alpha, Bm, in, (rocblas_int)ldb, A, in, (rocblas_int)lda, &beta, C, out,
                                            (rocblas_int)ldc, C, out, (rocblas_int)ldc, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
  if (st != rocblas_status_success) return fail(RTN_ERR_HIP, "rocblas_gemm_ex failed with status %d", (int)st);
  return RTN_OK;
}

struct BwdLayout {
  size_t off_sync = 0, off_dyw = 0, off_dx0 = 0, off_wpk = 0, off_ex = 0, total = 0;  // [0, off_wpk) is cleared at the start of a call
};
BwdLayout bwd_layout(int B, int n, int dtype) {
  BwdLayout l;
  size_t off = 256;  // status block, as in the forward workspace
  l.off_sync = off;  // two words per batch group (at most B groups): the XCD check of the persistent kernel
  off = align_up(off + (size_t)B * 8, 256);
  l.off_dyw = off;
  off = align_up(off + (size_t)B * n * 4, 256);
  l.off_dx0 = off;
  off = align_up(off + (size_t)B * 4 * n * esize(dtype), 256);
  l.off_wpk = off;  // W in fragment order, for per-frame launches
  if (n % 16 == 0) off = align_up(off + (size_t)4 * n * n * esize(dtype), 256);
  // the exchange ring of the persistent kernel: kExRing frames of 4n x Bp elements per batch group; groups of at least 4
  // rows in frames of 8, or of more than 8 rows in frames of 16: never more than 2B + 16 rows in all
  l.off_ex = off;
  if (n % 16 == 0) off = align_up(off + (size_t)kExRing * 4 * n * esize(dtype) * (2 * (size_t)B + 16), 256);
  l.total = off;
  return l;
}

typedef void (*SeqKernel)(float*, int);
template <typename AT>
SeqKernel seq_kernel_for(int MT, int NT, int KSMAX, bool half) {
  // the decompositions of the benchmark configurations and their neighbours
  if (half) {
    if (MT == 8 && NT == 1 && KSMAX == 8) return &k_mfma_sequence<AT, 8, 1, 8, true>;
    if (MT == 4 && NT == 1 && KSMAX == 8) return &k_mfma_sequence<AT, 4, 1, 8, true>;
    if (MT == 4 && NT == 1 && KSMAX == 4) return &k_mfma_sequence<AT, 4, 1, 4, true>;
    return nullptr;
  }
  if (MT == 8 && NT == 1 && KSMAX == 8) return &k_mfma_sequence<AT, 8, 1, 8, false>;
  if (MT == 4 && NT == 1 && KSMAX == 8) return &k_mfma_sequence<AT, 4, 1, 8, false>;
  if (MT == 2 && NT == 1 && KSMAX == 8) return &k_mfma_sequence<AT, 2, 1, 8, false>;
  if (MT == 1 && NT == 1 && KSMAX == 2) return &k_mfma_sequence<AT, 1, 1, 2, false>;
  return nullptr;
}

// The matrix cores alone on the plan's tile sequence (k_mfma_issue): same decompositions as the sequence probe.
template <typename AT>
SeqKernel issue_kernel_for(int MT, int NT, int KSMAX) {
  if (MT == 8 && NT == 1 && KSMAX == 8) return &k_mfma_issue<AT, 8, 1, 8>;
  if (MT == 4 && NT == 1 && KSMAX == 8) return &k_mfma_issue<AT, 4, 1, 8>;
  if (MT == 4 && NT == 1 && KSMAX == 4) return &k_mfma_issue<AT, 4, 1, 4>;
  if (MT == 2 && NT == 1 && KSMAX == 8) return &k_mfma_issue<AT, 2, 1, 8>;
  if (MT == 1 && NT == 1 && KSMAX == 2) return &k_mfma_issue<AT, 1, 1, 2>;
  return nullptr;
}

// Both measurement probes: the plan's grid runs `steps` steps of the plan's MFMA tile sequence -- with the partial tiles
// through LDS, the step's barrier and their sum (the decomposition's own ceiling), or the MFMAs alone (issue_only).
int mfma_probe(bool issue_only, int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t steps, void* workspace,
               size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (count < 1 || steps < 1 || steps > (1 << 24)) return fail(RTN_ERR_ARG, "MFMA sequence probe: count and steps must be positive");
  Plan pl;
  std::string why;
  const int c = std::min<int>(count, kMaxMulti);
  if (!make_plan(T, B, n, dtype, RTN_MODE_PERSISTENT, false, &pl, &why, 2, c) || !pl.regw)
    return fail(RTN_ERR_UNSUPPORTED, "MFMA sequence probe: the shape has no persistent register-kernel plan (%s)", why.c_str());
  SeqKernel k;
  int threads = kWgThreads;
  if (issue_only && env_long("RTN_LSTM2_PROBE_WAVES", 4) == 8 && dtype == RTN_DTYPE_BF16 && pl.MT == 8 && pl.NT == 1 && pl.KSMAX == 8) {
    // measurement variant: the same MFMAs dealt to two wavefronts per SIMD (eight per workgroup, 32 MFMAs each) -- what
    // the matrix cores do when a second wavefront fills the gaps one wavefront leaves between its MFMAs
    k = &k_mfma_issue<__bf16, 8, 1, 4, 512>;
    threads = 512;
  } else if (issue_only && env_long("RTN_LSTM2_PROBE_OTHERS", 0) > 0 && dtype == RTN_DTYPE_BF16 && pl.MT == 8 && pl.NT == 1 && pl.KSMAX == 8) {
    // measurement variant: one, two or three vector instructions behind every MFMA -- how much of a step's other work a
    // wavefront can issue in the MFMAs' shadow
    const long others = env_long("RTN_LSTM2_PROBE_OTHERS", 0);
    k = others == 1 ? &k_mfma_issue<__bf16, 8, 1, 8, kWgThreads, 1> : others == 2 ? &k_mfma_issue<__bf16, 8, 1, 8, kWgThreads, 2> : &k_mfma_issue<__bf16, 8, 1, 8, kWgThreads, 3>;
  } else if (issue_only)
    k = dtype == RTN_DTYPE_BF16 ? issue_kernel_for<__bf16>(pl.MT, pl.NT, pl.KSMAX) : issue_kernel_for<float>(pl.MT, pl.NT, pl.KSMAX);
  else
    k = dtype == RTN_DTYPE_BF16 ? seq_kernel_for<__bf16>(pl.MT, pl.NT, pl.KSMAX, pl.half) : seq_kernel_for<float>(pl.MT, pl.NT, pl.KSMAX, pl.half);
  if (!k) return fail(RTN_ERR_UNSUPPORTED, "MFMA sequence probe: no build for mt=%d nt=%d ks=%d", pl.MT, pl.NT, pl.KSMAX);
  // the workgroups that do the plan's work: an XCD-local grid is dealt over all XCDs and part of it may leave at once
  const int wgs = pl.local ? c * pl.groups * pl.wgs_per_group : (c == 1 ? pl.grid : pl.grid * c);
  const size_t need = (size_t)wgs * kWgThreads * sizeof(float);
  if (!workspace || workspace_bytes < need) return fail(RTN_ERR_WORKSPACE, "MFMA sequence probe: workspace of %zu bytes needed", need);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "MFMA sequence probe: workspace must be 16-byte aligned");
  const size_t lds = issue_only ? 0 : (size_t)2 * kWaves * pl.MT * pl.NT * kTileBytes + (size_t)kWaves * pl.KSMAX * pl.NT * kTileBytes;
  rc = ensure_lds_limit((const void*)k, lds);
  if (rc != RTN_OK) return rc;
  float* out = (float*)workspace;
  int st = steps;
  void* args[] = {(void*)&out, (void*)&st};
  RTN_HIP(hipLaunchKernel((const void*)k, dim3((unsigned)wgs), dim3((unsigned)threads), args, lds, (hipStream_t)hip_stream));
  return RTN_OK;
}

// Device address of this GPU's copy of `scratch`: asked of the runtime once per device, with that device current.
int static_scratch(void** out) {
  static std::mutex mu;
  static void* ptrs[64] = {nullptr};
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(RTN_ERR_HIP, "NativeLstm2: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* ptr = nullptr;
    RTN_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(RTN_ERR_HIP, "NativeLstm2: the runtime gave no address for the static scratch array");
    ptrs[dev] = ptr;
  }
  *out = ptrs[dev];
  return RTN_OK;
}

}  // namespace
}  // namespace rtn

using namespace rtn;

extern "C" {

int rtn_native_lstm2_abi_version(void) { return 13; }

const char* rtn_native_lstm2_bwd_plan_text(void) { return g_bwd_plan_text.c_str(); }

void rtn_native_lstm2_reload_env(void) { reload_env(); }

const char* rtn_native_lstm2_capture_report(void) {
  static thread_local std::string text;
  std::lock_guard<std::mutex> lock(g_capture_mu);
  char buf[256];
  snprintf(buf, sizeof(buf), "persistent launches recorded under stream capture: %lld as cooperative kernel nodes, %lld as ordinary kernel nodes",
           g_capture_cooperative, g_capture_plain);
  text = buf;
  if (!g_capture_refusal.empty()) text += "; cooperative node refused by " + g_capture_refusal;
  return text.c_str();
}

int rtn_graph_cache_stats(int64_t* out, int32_t n_out) {
  g_last_error.clear();
  if (!out || n_out < 5) return fail(RTN_ERR_ARG, "NativeLstm2: the graph statistics need room for 5 numbers");
  std::lock_guard<std::mutex> lock(g_graph_mu);
  sweep_retired();
  out[0] = (int64_t)g_graphs.size();
  out[1] = (int64_t)g_retired.size();
  out[2] = g_graph_records;
  out[3] = g_graph_retargets;
  out[4] = g_graph_destroyed;
  return RTN_OK;
}

const char* rtn_last_error(void) { return g_last_error.c_str(); }

size_t rtn_native_lstm2_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  if (check_dims(T, B, n, dtype) != RTN_OK) return 0;
  if (mode < RTN_MODE_AUTO || mode > RTN_MODE_STEPWISE) return 0;
  return workspace_each(1, T, B, n, dtype, mode);
}

const char* rtn_native_lstm2_describe_multi_plan(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  Plan pl;
  std::string why;
  char buf[512];
  const int c = env_long("RTN_LSTM2_NO_FUSE", 0) ? 1 : std::max(1, std::min(count, kMaxMulti));
  const int n_asked = n;
  if (check_dims(T, B, n, dtype) == RTN_OK && T > 0 && B > 0) n = padded_width(n);  // the plan is that of the padded problem
  if (check_dims(T, B, n, dtype) != RTN_OK) {
    g_plan_text = "invalid: " + g_last_error;
  } else if (!make_plan(T, B, n, dtype, mode, false, &pl, &why, 2, c)) {
    g_plan_text = "unsupported: " + why;
  } else {
    snprintf(buf, sizeof(buf), "mode=%s kernel=%s mt=%d nt=%d groups=%d wgs_per_group=%d wgs=%d rows_per_group=%d launches=%d lds=%zu workspace=%zu",
             mode_name(pl.mode),
             pl.kind == kPlanMfma ? (pl.regw ? (pl.local ? (pl.half ? "mfma_regw_xcd_half" : "mfma_regw_xcd") : "mfma_regw") : "mfma_lds") : (pl.kind == kPlanGeneric ? "generic" : "empty"), pl.MT,
             pl.NT, pl.groups, pl.wgs_per_group, (pl.mode == RTN_MODE_PERSISTENT && pl.regw) ? pl.grid : pl.groups * pl.wgs_per_group,
             pl.Bg, pl.passes, pl.lds_bytes,
             (count > 1 || n != n_asked) ? workspace_each(count, T, B, n_asked, dtype, mode) : pl.total);
    if (n != n_asked) snprintf(buf + strlen(buf), sizeof(buf) - strlen(buf), " padded_width=%d", n);
    if (pl.off_trace) snprintf(buf + strlen(buf), sizeof(buf) - strlen(buf), " trace_offset=%zu", pl.off_trace);
    g_plan_text = buf;
  }
  return g_plan_text.c_str();
}

const char* rtn_native_lstm2_describe_plan(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  return rtn_native_lstm2_describe_multi_plan(1, T, B, n, dtype, mode);
}

int rtn_native_lstm2_fwd(const void* X, const void* W, const void* y0, const float* c0, const float* i, int32_t start,
                         int32_t step, void* Y, float* C, void* H, float* d, int64_t T, int32_t B, int32_t n,
                         int32_t dtype, int32_t mode, void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  rtn_lstm2_call call = {X, W, y0, c0, i, start, step, Y, C, H, d};
  return fwd_calls(&call, 1, T, B, n, dtype, mode, workspace, workspace_bytes, hip_stream);
}

int rtn_native_lstm2_fwd_static(const void* X, const void* W, const void* y0, const float* c0, const float* i, int32_t start,
                                int32_t step, void* Y, float* C, void* H, float* d, int64_t T, int32_t B, int32_t n,
                                int32_t dtype, int32_t mode, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (mode < RTN_MODE_AUTO || mode > RTN_MODE_STEPWISE) return fail(RTN_ERR_ARG, "NativeLstm2: unknown mode %d", mode);
  if (mode == RTN_MODE_GRAPH)
    return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2: GRAPH mode replays a library-owned graph, which has to be created; "
                "the entry that allocates nothing takes AUTO, PERSISTENT or STEPWISE");
  const size_t need = workspace_each(1, T, B, n, dtype, mode);
  if (need > (size_t)RTN_STATIC_SCRATCH_BYTES)
    return fail(RTN_ERR_WORKSPACE, "NativeLstm2: T=%lld B=%d n=%d needs %zu bytes of scratch, the static array holds %zu; "
                "use rtn_native_lstm2_fwd with a workspace", (long long)T, B, n, need, (size_t)RTN_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != RTN_OK) return rc;
  rtn_lstm2_call call = {X, W, y0, c0, i, start, step, Y, C, H, d};
  // (nothing may be created at call time here: the persistent kernel keeps the cooperative launch, which needs no event)
  g_no_setup_objects = true;
  rc = fwd_calls(&call, 1, T, B, n, dtype, mode, ws, (size_t)RTN_STATIC_SCRATCH_BYTES, hip_stream, 0, 0, /*no_graph=*/true);
  g_no_setup_objects = false;
  return rc;
}

int rtn_native_lstm2_fwd_multi(const rtn_lstm2_call* calls, int32_t count, int64_t T, int32_t B, int32_t n,
                               int32_t dtype, int32_t mode, void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  if (count < 0 || (count > 0 && !calls)) return fail(RTN_ERR_ARG, "NativeLstm2: bad call list (count=%d)", count);
  if (count == 0) return RTN_OK;
  return fwd_calls(calls, count, T, B, n, dtype, mode, workspace, workspace_bytes, hip_stream);
}

int rtn_handover_latency_probe(void* workspace, size_t workspace_bytes, int32_t rounds, void* hip_stream) {
  g_last_error.clear();
  constexpr int G = 16;
  const size_t need = 256 + (size_t)4 * G * 256;
  if (!workspace || workspace_bytes < need) return fail(RTN_ERR_WORKSPACE, "handover probe: workspace of %zu bytes needed", need);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "handover probe: workspace must be 16-byte aligned");
  if (rounds < 1 || rounds > (1 << 24)) return fail(RTN_ERR_ARG, "handover probe: rounds must be in [1, 2^24]");
  if (!device_info().cooperative || device_info().cus < G) return fail(RTN_ERR_UNSUPPORTED, "handover probe: needs cooperative launch and %d CUs", G);
  hipStream_t stream = (hipStream_t)hip_stream;
  unsigned* status = (unsigned*)workspace;
  unsigned* ring = (unsigned*)((unsigned char*)workspace + 256);
  const long long words = (long long)(need / 4);
  hipLaunchKernelGGL(k_fill_u32, dim3(8), dim3(256), 0, stream, (unsigned*)workspace, 0u, words);
  RTN_HIP(hipGetLastError());
  int g = G, rnd = rounds;
  unsigned long long ticks = (unsigned long long)env_long("RTN_LSTM2_TIMEOUT_TICKS", 200000000L);
  void* args[] = {(void*)&ring, (void*)&status, (void*)&g, (void*)&rnd, (void*)&ticks};
  RTN_HIP(hipLaunchCooperativeKernel((const void*)k_handover_latency, dim3(G), dim3(kWgThreads), args, 0, stream));
  return RTN_OK;
}

int rtn_mfma_sequence_probe(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t steps, void* workspace,
                            size_t workspace_bytes, void* hip_stream) {
  return mfma_probe(false, count, T, B, n, dtype, steps, workspace, workspace_bytes, hip_stream);
}

int rtn_mfma_issue_probe(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t steps, void* workspace,
                         size_t workspace_bytes, void* hip_stream) {
  return mfma_probe(true, count, T, B, n, dtype, steps, workspace, workspace_bytes, hip_stream);
}

size_t rtn_native_lstm2_fwd_multi_workspace_bytes(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  if (count < 0 || check_dims(T, B, n, dtype) != RTN_OK) return 0;
  if (mode < RTN_MODE_AUTO || mode > RTN_MODE_STEPWISE) return 0;
  return (size_t)count * workspace_each(count, T, B, n, dtype, mode);
}

int rtn_native_lstm2_fwd_multi_status(const void* workspace, int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype,
                                      int32_t mode, void* hip_stream) {
  g_last_error.clear();
  if (check_dims(T, B, n, dtype) != RTN_OK || mode < RTN_MODE_AUTO || mode > RTN_MODE_STEPWISE) return RTN_ERR_ARG;
  const size_t each = workspace_each(std::max(count, 1), T, B, n, dtype, mode);  // call k's slice starts at k * each
  if (!workspace || each == 0 || count < 0) return fail(RTN_ERR_ARG, "NativeLstm2: bad arguments to the status query");
  for (int k = 0; k < count; ++k) {
    const int rc = rtn_native_lstm2_fwd_status((const unsigned char*)workspace + (size_t)k * each, hip_stream);
    if (rc != RTN_OK) return rc;
  }
  return RTN_OK;
}

size_t rtn_lstm_generic_base_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode) {
  const size_t fwd = rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode);
  if (fwd == 0) return 0;
  // forward workspace | zero initial output [B,n] | cell states [T,B,n] float32 (the op has no C output)
  return fwd + align_up((size_t)B * n * esize(dtype), 256) + align_up((size_t)T * B * n * 4, 256);
}

int rtn_lstm_generic_base_fwd(const void* Z, const void* V_h, const float* c, const float* i, void* Y, void* H, float* d,
                              int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode, void* workspace,
                              size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (T == 0) return fail(RTN_ERR_SHAPE, "LstmGenericBase: needs T > 0");  // returnn/native_op.py:504
  const size_t need = rtn_lstm_generic_base_fwd_workspace_bytes(T, B, n, dtype, mode);
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "LstmGenericBase: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "LstmGenericBase: workspace must be 16-byte aligned");
  const size_t fwd = rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode);
  unsigned char* ws = (unsigned char*)workspace;
  void* y0 = ws + fwd;
  const size_t y0_bytes = align_up((size_t)B * n * esize(dtype), 256);
  float* C = (float*)(ws + fwd + y0_bytes);
  if ((long long)B * n > 0) {
    hipLaunchKernelGGL(k_fill_u32, dim3(64), dim3(256), 0, (hipStream_t)hip_stream, (unsigned*)y0, 0u, (long long)(y0_bytes / 4));
    RTN_HIP(hipGetLastError());
  }
  rtn_lstm2_call call = {Z, V_h, y0, c, i, 0, 1, Y, C, H, d};
  return fwd_calls(&call, 1, T, B, n, dtype, mode, workspace, fwd, hip_stream, kOpNoCarry | kOpH0IsCell);
}

size_t rtn_lstm_low_mem_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype, int32_t mode) {
  (void)n_in;
  const size_t fwd = rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode);
  if (fwd == 0) return 0;
  // forward workspace | projected input [T,B,4n] | activated gates [T,B,4n] (the op has no H output)
  return fwd + 2 * align_up((size_t)T * B * 4 * n * esize(dtype), 256);
}

int rtn_lstm_low_mem_fwd(const void* X, const void* W, const void* b, const void* y0, const float* c0, const float* i,
                         int32_t start, int32_t step, void* Y, float* C, float* d, int64_t T, int32_t B, int32_t n_in,
                         int32_t n, int32_t dtype, int32_t mode, void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (n_in < 0) return fail(RTN_ERR_SHAPE, "LstmLowMem: negative input dimension %d", n_in);
  if (T > 0 && (long long)B * n > 0 && step < 0 && start >= 0 && start < T && T - start - 1 < start)
    return fail(RTN_ERR_RANGE, "LstmLowMem: start=%d with a negative step visits no frame of T=%lld", start, (long long)T);
  hipStream_t stream = (hipStream_t)hip_stream;
  hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
  if (stream) RTN_HIP(hipStreamIsCapturing(stream, &cap_status));
  (void)cap_status;  // under capture the rocBLAS projection is recorded like the launches (the handle must exist already)
  const size_t need = rtn_lstm_low_mem_fwd_workspace_bytes(T, B, n_in, n, dtype, mode);
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "LstmLowMem: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "LstmLowMem: workspace must be 16-byte aligned");
  const size_t es = esize(dtype);
  const size_t fwd = rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode);
  const size_t frame_bytes = align_up((size_t)T * B * 4 * n * es, 256);
  unsigned char* ws = (unsigned char*)workspace;
  void* Xp = ws + fwd;
  void* Hs = ws + fwd + frame_bytes;
  const long long rows = (long long)T * B;
  const unsigned char* W_rec = (const unsigned char*)W + (size_t)n_in * 4 * n * es;  // rows n_in.. of W: the recurrent part
  if (rows > 0 && n > 0) {
    if (!X || !W || !b) return fail(RTN_ERR_ARG, "LstmLowMem: X, W and b must not be null");
    if (!aligned16(W)) return fail(RTN_ERR_ARG, "LstmLowMem: W must be 16-byte aligned");
    // Xp = X . W[:n_in] + b   (returnn/native_op.py:815-826, the part of `intern` that does not depend on the recurrence)
    rocblas_handle blas = nullptr;
    rc = blas_handle(&blas);
    if (rc != RTN_OK) return rc;
    if (rocblas_set_stream(blas, stream) != rocblas_status_success) return fail(RTN_ERR_HIP, "LstmLowMem: rocblas_set_stream failed");
    const rocblas_datatype ty = dtype == RTN_DTYPE_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f32_r;
    if (n_in > 0) {
      const float alpha = 1.f, beta = 0.f;
      // row-major Xp[rows,4n] = column-major [4n,rows] = W_ff (column-major [4n,n_in]) * X (column-major [n_in,rows])
      const rocblas_status st = rocblas_gemm_ex(blas, rocblas_operation_none, rocblas_operation_none, 4 * n, (rocblas_int)rows, n_in, &alpha, W, ty,
                                                4 * n, X, ty, n_in, &beta, Xp, ty, 4 * n, Xp, ty, 4 * n, rocblas_datatype_f32_r,
                                                rocblas_gemm_algo_standard, 0, 0);
      if (st != rocblas_status_success) return fail(RTN_ERR_HIP, "LstmLowMem: rocblas_gemm_ex failed with status %d", (int)st);
    } else {
      hipLaunchKernelGGL(k_fill_u32, dim3(1024), dim3(256), 0, stream, (unsigned*)Xp, 0u, (long long)(frame_bytes / 4));
    }
    const long long total = rows * 4 * n;
    const dim3 grid((unsigned)std::min<long long>((total + 255) / 256, 65535)), block(256);
    if (dtype == RTN_DTYPE_BF16)
      hipLaunchKernelGGL(k_add_bias<__bf16>, grid, block, 0, stream, Xp, b, total, 4 * n);
    else
      hipLaunchKernelGGL(k_add_bias<float>, grid, block, 0, stream, Xp, b, total, 4 * n);
    RTN_HIP(hipGetLastError());
  }
  rtn_lstm2_call call = {Xp, W_rec, y0, c0, i, start, step, Y, C, Hs, d};
  // With a negative step the reference's loop ends at frame `start`, and for 2*start > T-1 it visits no frame and
  // returns an uninitialised d (returnn/native_op.py:827-833, :834); that case is refused with RTN_ERR_RANGE.
  return fwd_calls(&call, 1, T, B, n, dtype, mode, workspace, fwd, hip_stream, kOpNoCarry | kOpEndAtStart);
}

size_t rtn_native_lstm2_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype) {
  if (check_dims(T, B, n, dtype) != RTN_OK) return 0;
  const int np = padded_width(n);
  if (np == n || T == 0 || B == 0) return bwd_layout(B, n, dtype).total;
  // a padded width: the workspace of the padded problem, then the padded copies
  return bwd_layout(B, np, dtype).total + bwd_pad_layout(T, B, np, dtype).total;
}

namespace {

// Per-call state of the gradient entry between its three phases (prepare, recurrence, weight gradient).
struct BwdJob {
  Lstm2BwdParams p;
  unsigned char* ws;
  long long abs_step, num_steps, first, end;
  long long ldY;  // row pitch of Y in elements
};

// What all phases of one gradient entry share.
struct BwdCtx {
  const rtn_lstm2_bwd_call* calls;
  int count;
  int64_t T;
  int B, n, dtype, op_flags;
  hipStream_t stream;
  bool capturing;
  size_t es;     // bytes per activation element
  long long bn;  // B * n
};

// The persistent kernel and decomposition of a gradient entry (kernel == nullptr: launches per frame).
struct BwdChoice {
  const void* kernel = nullptr;
  int ksb = 0;                 // macro steps of the contraction per wavefront
  int tiles = 1;               // tiles of 16 values of k per workgroup
  int waves = kWaves;          // wavefronts per workgroup
  int rows_per_group = 16;     // batch rows per group
  int groups_per_launch = 0;   // batch groups of every problem that one launch takes
  bool local = false;          // every group on one XCD
  size_t lds = 0;              // dynamic shared memory of the kernel
};

int bwd_calls(const rtn_lstm2_bwd_call* calls, int count, int64_t T, int32_t B, int32_t n, int32_t dtype, void* workspace,
              size_t workspace_bytes, void* hip_stream, int op_flags = 0, size_t ws_stride = 0);

// Argument checks and the outputs that do not depend on the recurrence: DW := 0, Dc0 := Dd, and Dy0 := 0 where there is
// no frame to run (returnn/native_op.py:1365-1370).
int bwd_check_and_clear(const BwdCtx& x) {
  const long long nn4 = (long long)x.n * x.n * 4;
  const dim3 fill_grid(256), fill_block(256);
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    if (nn4 > 0 && !c.DW) return fail(RTN_ERR_ARG, "NativeLstm2 backward: DW must not be null");
    if (x.bn > 0 && (!c.Dd || !c.Dy0 || !c.Dc0)) return fail(RTN_ERR_ARG, "NativeLstm2 backward: Dd, Dy0 and Dc0 must not be null");
  }
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    if (nn4 > 0) {
      hipLaunchKernelGGL(k_fill_u32, fill_grid, fill_block, 0, x.stream, (unsigned*)c.DW, 0u, nn4);
      RTN_HIP(hipGetLastError());
    }
    if (x.bn > 0) {
      hipLaunchKernelGGL(k_copy_f32, fill_grid, fill_block, 0, x.stream, c.Dd, c.Dc0, x.bn);
      RTN_HIP(hipGetLastError());
    }
    if ((x.T == 0 || x.bn == 0) && x.bn > 0) {
      hipLaunchKernelGGL(k_fill_u32, fill_grid, fill_block, 0, x.stream, (unsigned*)c.Dy0, 0u, (long long)(((size_t)x.bn * x.es + 3) / 4));
      RTN_HIP(hipGetLastError());
    }
  }
  if (x.T == 0 || x.bn == 0 || x.count == 0) return RTN_OK;
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    if (c.start < 0 || c.start >= x.T)
      return fail(RTN_ERR_RANGE, "NativeLstm2 backward: need 0 <= start < T, got start=%d, T=%lld", c.start, (long long)x.T);
    if (c.step == 0) return fail(RTN_ERR_RANGE, "NativeLstm2 backward: step must not be 0");
    const void* ptrs[] = {c.W, c.y0, c.c0, c.i, c.Y, c.C, c.H, c.DY, c.Dd, c.DX, c.DW, c.Dy0, c.Dc0};
    const char* names[] = {"W", "y0", "c0", "i", "Y", "C", "H", "DY", "Dd", "DX", "DW", "Dy0", "Dc0"};
    for (int q = 0; q < 13; ++q) {
      if (!ptrs[q]) return fail(RTN_ERR_ARG, "NativeLstm2 backward: %s must not be null", names[q]);
      // (W is read in 16-byte fragments only where n is a multiple of 16; the recurrent rows of a stacked matrix start at
      // a multiple of 4n elements, which is aligned then)
      if (q != 3 && !(q == 0 && x.n % 16 != 0) && !aligned16(ptrs[q])) return fail(RTN_ERR_ARG, "NativeLstm2 backward: %s must be 16-byte aligned", names[q]);
    }
  }
  return RTN_OK;
}

// The problem zero-padded to a width the matrix-core kernels take (see padded_width), on copies in the workspace: slice
// k = the workspace of the padded call k, then its copies.
int bwd_padded(const BwdCtx& x, int np, void* workspace, size_t workspace_bytes) {
  const int n = x.n, B = x.B;
  const BwdLayout lay_p = bwd_layout(B, np, x.dtype);
  const BwdPadLayout L = bwd_pad_layout(x.T, B, np, x.dtype);
  const size_t each = lay_p.total + L.total;
  const size_t need = (size_t)x.count * each;
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "NativeLstm2 backward: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "NativeLstm2 backward: workspace must be 16-byte aligned");
  const size_t es = x.es;
  const long long tb = (long long)x.T * B;
  int rc = RTN_OK;
  std::vector<rtn_lstm2_bwd_call> padded((size_t)x.count);
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    unsigned char* base = (unsigned char*)workspace + (size_t)k * each + lay_p.total;
    if ((rc = launch_pad(c.W, base + L.W, n, np, 4, n, np, es, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.y0, base + L.y0, B, B, 1, n, np, es, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.c0, base + L.c0, B, B, 1, n, np, 4, x.stream)) != RTN_OK) return rc;
    long long ldY = 0, ldDY = 0, ldDX = 0;
    if ((rc = resolve_pitch("ldY", c.ldY, n, B, es, &ldY)) != RTN_OK) return rc;
    if ((rc = resolve_pitch("ldDY", c.ldDY, n, B, es, &ldDY)) != RTN_OK) return rc;
    if ((rc = resolve_pitch("ldDX", c.ldDX, 4LL * n, B, es, &ldDX)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.Y, base + L.Y, tb, tb, 1, n, np, es, x.stream, ldY)) != RTN_OK) return rc;
    // the sibling op that keeps its cell states in H hands H in for C as well; it is not read then
    if (!(x.op_flags & kOpH0IsCell) && (rc = launch_pad(c.C, base + L.C, tb, tb, 1, n, np, 4, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.H, base + L.H, tb, tb, 4, n, np, es, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.DY, base + L.DY, tb, tb, 1, n, np, es, x.stream, ldDY)) != RTN_OK) return rc;
    if ((rc = launch_pad(c.Dd, base + L.Dd, B, B, 1, n, np, 4, x.stream)) != RTN_OK) return rc;
    padded[(size_t)k] = {base + L.W, base + L.y0, (const float*)(base + L.c0), c.i, c.start, c.step, base + L.Y,
                         (const float*)(base + ((x.op_flags & kOpH0IsCell) ? L.H : L.C)), base + L.H, base + L.DY,
                         (const float*)(base + L.Dd), base + L.DX, (float*)(base + L.DW), base + L.Dy0, (float*)(base + L.Dc0),
                         0, 0, 0};
  }
  rc = bwd_calls(padded.data(), x.count, x.T, B, np, x.dtype, workspace, need, (void*)x.stream, x.op_flags, each);
  if (rc != RTN_OK) return rc;
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    const rtn_lstm2_bwd_call& q = padded[(size_t)k];
    if ((rc = launch_unpad(q.DX, c.DX, tb, 4, n, np, es, x.stream, c.ldDX)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.DW, c.DW, n, 4, n, np, 4, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.Dy0, c.Dy0, B, 1, n, np, es, x.stream)) != RTN_OK) return rc;
    if ((rc = launch_unpad(q.Dc0, c.Dc0, B, 1, n, np, 4, x.stream)) != RTN_OK) return rc;
  }
  return RTN_OK;
}

// Persistent kernel: W in registers for the whole call, if a wavefront's share of the 16 x 4n slice fits (2..32
// fragments, 64 with half of them in LDS) and all workgroups of all problems can be on the device together.
// Decomposition: batch groups of 4, 8 or 16 rows (a workgroup's frame time grows with the rows x 4n derivatives it reads
// per frame from the exchange ring), 1, 2 or 4 tiles of 16 values of k per workgroup (more tiles: fewer workgroups, more
// MFMA time each) and 4 or 8 wavefronts per workgroup.  Leaves out->kernel null where no candidate fits.
int choose_bwd_kernel(const BwdCtx& x, BwdChoice* out) {
  const int n = x.n, B = x.B, dtype = x.dtype, count = x.count;
  int rc = RTN_OK;
  BwdChoice best, turn;  // turn: the candidate that takes most rows per launch, for batches that need several launches
  long long turn_rows = 0;
  const int KM = dtype == RTN_DTYPE_BF16 ? 32 : 16;
  const int S = 4 * n / KM;
  const long env_rows = env_long("RTN_LSTM2_BWD_ROWS", 0);
  const long env_mt = env_long("RTN_LSTM2_BWD_MT", 0);
  const long env_waves = env_long("RTN_LSTM2_BWD_WAVES", 0);
  // (rows per group, tiles per workgroup, wavefronts per workgroup, XCD-local only)
  // Candidates in the order measured on MI355X (cfg3 bf16 n=1024, ms per gradient call: one problem 8 x 1 x 4: 2.73,
  // 8 x 1 x 8: 3.04, 8 x 2 x 4 on one XCD per group: 3.2, 16 x 1 x 8: 3.6; two problems in one launch 8 x 2 x 4 on one
  // XCD per group: 3.53, spread: 3.78; cfg2 float32 n=512: 8 x 1 x 4 on one XCD per group 2.35, spread 2.56, 8 x 1 x 8:
  // 2.55 / 2.79, 8 x 2 x 4: 3.4); the first whose workgroups are all on the device together.  A candidate whose groups
  // fit an XCD each (n / (16 * tiles) workgroups, all groups of all problems in one launch) runs XCD-local: the ring
  // then goes from writer to readers through that XCD's L2 instead of through memory.
  // In front of them, for bf16 only and only where its groups fit an XCD each: 4 rows x 2 tiles, the kernel with one
  // (row, k) pair per thread (one problem of cfg3: 4.82 ms against 5.03 for 8 x 1 x 4, whose groups of 64 workgroups
  // span two XCDs; in float32 two tiles double an MFMA time that is long already: cfg2 3.1 ms against 2.3).
  const int candidates[][4] = {{4, 2, 4, 1}, {8, 1, 4, 0}, {8, 1, 8, 0}, {8, 2, 4, 0}, {16, 1, 4, 0}, {16, 1, 8, 0}, {16, 2, 4, 0}, {8, 4, 4, 0}, {16, 4, 4, 0}};
  const DeviceInfo di = device_info();
  const long want_local = env_long("RTN_LSTM2_BWD_LOCAL", 1);
  for (const auto& cand : candidates) {
    const int rows = cand[0], mt = cand[1];
    const int wv = env_waves ? (int)env_waves : cand[2];
    const bool local_only = cand[3] != 0;
    if (local_only && (dtype != RTN_DTYPE_BF16 || env_mt || env_waves || (env_rows >= 1 && env_rows <= 16))) continue;
    if (env_mt && mt != env_mt) continue;
    const bool rows_forced = env_rows >= 1 && env_rows <= 16;  // an explicit row count replaces the candidates' own
    if (rows_forced && rows != 8) continue;                    // (one pass per MT is enough then)
    const int use_rows = rows_forced ? (int)env_rows : rows;
    if (wv != 4 && wv != 8 && wv != 16) continue;
    const int ksb = (S + wv - 1) / wv;  // macro steps per wavefront; the kernel has room for the next power of two
    int ksb_room = 2;
    while (ksb_room < ksb) ksb_room *= 2;
    if (mt * ksb_room > 64 || (n / 16) % mt) continue;
    // A share of 64 fragments does not fit the registers next to a frame's DX (with all of it in registers the compiler
    // spills part of W, in float32 most of it): half of it lives in LDS.
    const bool lds_share = ksb_room * wv == 256;
    if (lds_share && (mt != 1 || (wv != 4 && wv != 8))) continue;
    BwdRegwKernel kfn;
    if (lds_share)
      kfn = dtype == RTN_DTYPE_BF16 ? bwd_regw_lds_table_bf16(wv) : bwd_regw_lds_table_f32(wv);
    else
      // ring frames of 8 rows: the variant whose loads take two macro steps at once
      kfn = use_rows <= 8 ? (dtype == RTN_DTYPE_BF16 ? bwd_regw_table_bf16_half(ksb_room, mt, wv) : bwd_regw_table_f32_half(ksb_room, mt, wv))
                          : (dtype == RTN_DTYPE_BF16 ? bwd_regw_table_bf16_full(ksb_room, mt, wv) : bwd_regw_table_f32_full(ksb_room, mt, wv));
    if (!kfn) continue;
    BwdChoice c;
    c.kernel = (const void*)kfn;
    c.ksb = ksb;
    c.tiles = mt;
    c.waves = wv;
    c.rows_per_group = use_rows;
    c.lds = lds_share ? kBwdLdsShareBytes : 0;
    if (c.lds && (rc = ensure_lds_limit(c.kernel, c.lds)) != RTN_OK) return rc;
    int per_cu = 0;
    if ((rc = occupancy_per_cu(c.kernel, 64 * wv, c.lds, &per_cu)) != RTN_OK) return rc;
    const long long groups_needed = (B + use_rows - 1) / use_rows;
    const long long G_wgs = n / (16 * mt), cu_x = di.xcds > 0 ? di.cus / di.xcds : 0;
    if (local_only && n / 16 <= cu_x * per_cu) continue;  // (groups of one tile per workgroup fit an XCD themselves)
    if (local_only && 2 * (long long)count * groups_needed * G_wgs < di.cus) continue;  // (few rows: the wider spread wins, cfg5 7.98 against 8.41 ms)
    const bool fits_xcd = want_local && di.xcds > 1 && per_cu >= 1 && G_wgs <= cu_x * per_cu;
    if (fits_xcd && (long long)di.xcds * ((cu_x * per_cu) / G_wgs) >= (long long)count * groups_needed) {
      c.groups_per_launch = (int)groups_needed;
      c.local = true;
      best = c;
      break;
    }
    if (local_only) continue;
    // batch groups of every problem that one launch can hold
    const long long fit = (long long)per_cu * di.cus / ((long long)count * G_wgs);
    if (fit >= groups_needed) {
      c.groups_per_launch = (int)groups_needed;
      best = c;
      break;
    }
    // Too many rows for one launch: remember the candidate that takes most rows per launch; the batch groups
    // then run in turns (the rows of a batch are independent of each other).  A turn whose groups fit an XCD each
    // is an XCD-local launch, unless that costs more than an eighth of the groups a launch can hold.
    const long long fit_local = fits_xcd ? (long long)di.xcds * ((cu_x * per_cu) / G_wgs) / count : 0;
    const bool local_turns = fit_local >= 1 && fit_local * 8 >= fit * 7;
    const long long turn_fit = local_turns ? fit_local : fit;
    if (turn_fit >= 1 && turn_fit * use_rows > turn_rows &&
        (groups_needed + turn_fit - 1) / turn_fit <= env_long("RTN_LSTM2_MAX_PASSES", kMaxPassesOverSteps)) {
      turn_rows = turn_fit * use_rows;
      c.groups_per_launch = (int)turn_fit;
      c.local = local_turns;
      turn = c;
    }
  }
  *out = best.kernel ? best : turn;
  return RTN_OK;
}

// Fills in the kernels' parameter blocks: buffers, pitches, the frames the forward pass visited (returnn/native_op.py:
// 1383-1407), and puts each call's workspace slice into its starting state.
int bwd_prepare_jobs(const BwdCtx& x, const BwdChoice& ch, const BwdLayout& lay, void* workspace, size_t stride, std::vector<BwdJob>* jobs) {
  const int n = x.n, B = x.B;
  const int64_t T = x.T;
  const int bgroups = (B + ch.rows_per_group - 1) / ch.rows_per_group;
  const dim3 fill_grid(256), fill_block(256);
  int rc = RTN_OK;
  jobs->assign((size_t)x.count, BwdJob());
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    BwdJob& j = (*jobs)[(size_t)k];
    Lstm2BwdParams& p = j.p;
    memset(&p, 0, sizeof(p));
    p.W = c.W; p.c0 = c.c0; p.mask = c.i; p.C = c.C; p.H = c.H; p.DY = c.DY;
    p.DX = c.DX; p.Dc0 = c.Dc0;
    j.ws = (unsigned char*)workspace + (size_t)k * stride;
    p.dyw = (float*)(j.ws + lay.off_dyw);
    p.dx0 = j.ws + lay.off_dx0;
    p.T = T; p.B = B; p.n = n;
    p.op_flags = x.op_flags;
    if ((rc = resolve_pitch("ldY", c.ldY, n, B, x.es, &j.ldY)) != RTN_OK) return rc;
    if ((rc = resolve_pitch("ldDY", c.ldDY, n, B, x.es, &p.ldDY)) != RTN_OK) return rc;
    if ((rc = resolve_pitch("ldDX", c.ldDX, 4LL * n, B, x.es, &p.ldDX)) != RTN_OK) return rc;
    hipLaunchKernelGGL(k_fill_u32, fill_grid, fill_block, 0, x.stream, (unsigned*)j.ws, 0u, (long long)(lay.off_wpk / 4));
    RTN_HIP(hipGetLastError());
    j.abs_step = c.step > 0 ? c.step : -(long long)c.step;
    j.num_steps = (T - c.start + j.abs_step - 1) / j.abs_step;
    j.first = c.step > 0 ? c.start : T - c.start - 1;
    if ((x.op_flags & kOpEndAtStart) && c.step < 0) {
      // LstmLowMem: with a negative step the frames from T-start-1 down to `start` (returnn/native_op.py:957-963)
      if (j.first < c.start) return fail(RTN_ERR_RANGE, "LstmLowMem gradient: start=%d with a negative step visits no frame of T=%lld", c.start, (long long)T);
      j.num_steps = (j.first - c.start) / j.abs_step + 1;
    }
    j.end = j.first + (j.num_steps - 1) * c.step;  // inclusive
    if (ch.kernel) {
      // the exchange ring starts armed: all-ones words (the visited frames of DX are written by the kernel, the others
      // zeroed behind it)
      const int bp = ch.rows_per_group > 8 ? 16 : 8;
      const long long ring_words = (long long)((size_t)bgroups * kExRing * 4 * n * x.es * bp / 4);
      if ((size_t)ring_words * 4 > lay.total - lay.off_ex)
        return fail(RTN_ERR_WORKSPACE, "NativeLstm2 backward: internal: exchange ring of %lld bytes does not fit its section", ring_words * 4);
      hipLaunchKernelGGL(k_fill_u32, dim3(256), fill_block, 0, x.stream, (unsigned*)(j.ws + lay.off_ex), 0xFFFFFFFFu, ring_words);
      RTN_HIP(hipGetLastError());
    } else if (j.num_steps != T) {
      // frames the loop does not visit keep DX = 0 (:1385-1388): all rows cleared here, row by row
      if ((rc = launch_clear_rows(c.DX, (long long)T * B, 4LL * n, p.ldDX, x.es, x.stream)) != RTN_OK) return rc;
    }
  }
  return RTN_OK;
}

// The recurrence of all problems on the persistent kernel: one launch per share of the batch groups (a single one unless
// the batch is too large for the device), then DX := 0 on the frames the forward pass did not visit.
int bwd_launch_persistent(const BwdCtx& x, const BwdChoice& ch, const BwdLayout& lay, const std::vector<BwdJob>& jobs) {
  const int n = x.n, B = x.B, count = x.count;
  const int bgroups = (B + ch.rows_per_group - 1) / ch.rows_per_group;
  const dim3 fill_block(256);
  Lstm2BwdMulti multi;
  memset(&multi, 0, sizeof(multi));
  multi.count = count;
  for (int k = 0; k < count; ++k) {
    Lstm2BwdPersistent& q = multi.q[k];
    const BwdJob& j = jobs[(size_t)k];
    q.p = j.p;
    q.Dd = x.calls[k].Dd;
    q.Dy0 = x.calls[k].Dy0;
    q.status = (unsigned*)j.ws;
    q.t_end = j.end;
    q.step = x.calls[k].step;
    q.nframes = (int)j.num_steps;
    q.Bg = (B + bgroups - 1) / bgroups;
    q.ksb = ch.ksb;
    // The kernels that keep one (row, k) pair per thread ask for a frame's inputs in front of the MFMAs, so only the
    // delay stands between a frame's stores and the read of its ring slot: inside an XCD it is a fixed one there, as in
    // the forward kernel (measured: 2.77 ms at 10 units against 2.82 adaptive and 2.87 / 2.86 at 4 / 16 for the layer).
    const bool one_pair = ch.rows_per_group <= 8 && ((ch.tiles + ch.waves / 4 - 1) / (ch.waves / 4)) % 2 == 0;
    const bool fixed_delay = ch.local && one_pair;
    q.poll_delay = (int)std::max<long>(0, std::min<long>(64, env_long("RTN_LSTM2_BWD_POLL_DELAY", fixed_delay ? 10 : 20)));
    q.delay_inc = (int)std::max<long>(0, std::min<long>(16, env_long("RTN_LSTM2_BWD_DELAY_INC", fixed_delay ? 0 : 2)));
    {
      long dec = env_long("RTN_LSTM2_BWD_DELAY_DEC", 16);  // steps per unit of downward adaptation: a power of two
      int mask = 0;
      while (2 * (mask + 1) <= dec && mask < 255) mask = 2 * mask + 1;
      q.delay_dec_mask = mask;
    }
    q.timeout_ticks = (unsigned long long)env_long("RTN_LSTM2_TIMEOUT_TICKS", 200000000L);
    q.sync = (unsigned*)(j.ws + lay.off_sync);
    q.ex = j.ws + lay.off_ex;
    q.Bp = ch.rows_per_group > 8 ? 16 : 8;
    q.bp_shift = ch.rows_per_group > 8 ? 4 : 3;
  }
  multi.local = ch.local ? 1 : 0;
  multi.xcds = device_info().xcds;
  const int wgs_per_group = n / (16 * ch.tiles);
  for (int g0 = 0; g0 < bgroups; g0 += ch.groups_per_launch) {
    const int groups_now = std::min(ch.groups_per_launch, bgroups - g0);
    multi.wgs_each = groups_now * wgs_per_group;
    for (int k = 0; k < count; ++k) {
      multi.q[k].groups = groups_now;
      multi.q[k].group_offset = g0;
    }
    void* args[] = {(void*)&multi};
    unsigned grid = (unsigned)(count * multi.wgs_each);
    if (ch.local) {
      // workgroup id = slot * xcds + xcd: the groups of the launch are dealt round-robin to the XCDs
      const int total_groups = count * groups_now;
      grid = (unsigned)(multi.xcds * wgs_per_group * ((total_groups + multi.xcds - 1) / multi.xcds));
    }
    const int rc = launch_coresident(ch.kernel, dim3(grid), dim3((unsigned)(64 * ch.waves)), args, (unsigned)ch.lds, x.stream, x.capturing);
    if (rc != RTN_OK) return rc;
  }
  for (int k = 0; k < count; ++k) {
    const BwdJob& j = jobs[(size_t)k];
    if (j.num_steps == x.T) continue;
    const long long row_words = (long long)((size_t)n * 4 * x.es / 4), pitch_words = (long long)((size_t)j.p.ldDX * x.es / 4);
    if (x.dtype == RTN_DTYPE_BF16)
      hipLaunchKernelGGL(k_bwd_zero_unvisited<__bf16>, dim3(1024), fill_block, 0, x.stream, x.calls[k].DX, (long long)x.T, (long long)B, row_words,
                         pitch_words, j.first, (long long)x.calls[k].step, j.num_steps);
    else
      hipLaunchKernelGGL(k_bwd_zero_unvisited<float>, dim3(1024), fill_block, 0, x.stream, x.calls[k].DX, (long long)x.T, (long long)B, row_words,
                         pitch_words, j.first, (long long)x.calls[k].step, j.num_steps);
    RTN_HIP(hipGetLastError());
  }
  return RTN_OK;
}

// The recurrence of ONE problem as launches per frame, in reverse processing order.  MFMA shapes: one fused launch per
// frame (the GEMM of the frame processed before, then this frame's pointwise part) and a last GEMM-only launch; other
// shapes: a pointwise and a generic GEMM launch per frame.  Replayed through a library-owned graph outside capture.
int bwd_launch_per_frame(const BwdCtx& x, bool mfma, const BwdLayout& lay, BwdJob& j) {
  const int n = x.n, B = x.B, dtype = x.dtype;
  hipStream_t stream = x.stream;
  if (mfma && env_long("RTN_LSTM2_BWD_PACK_W", 1)) {
    // every launch uses each fragment of W once: read them from a copy in fragment order (see k_bwd_pack_w)
    j.p.Wpk = j.ws + lay.off_wpk;
    const long long frags = (long long)(n / 16) * (4 * n / (dtype == RTN_DTYPE_BF16 ? 32 : 16)) * 64;
    const dim3 pgrid((unsigned)std::min<long long>((frags + 255) / 256, 4096)), pblock(256);
    if (dtype == RTN_DTYPE_BF16)
      hipLaunchKernelGGL(k_bwd_pack_w<__bf16>, pgrid, pblock, 0, stream, x.calls[0].W, (void*)j.p.Wpk, n);
    else
      hipLaunchKernelGGL(k_bwd_pack_w<float>, pgrid, pblock, 0, stream, x.calls[0].W, (void*)j.p.Wpk, n);
    RTN_HIP(hipGetLastError());
  }
  const Lstm2BwdParams& p = j.p;
  const int step = x.calls[0].step;
  const long long first = j.first, end = j.end;
  // Batch rows per workgroup (16 * NT): 32 if that still leaves every CU a workgroup (each batch tile reads W again),
  // else 16 (measured: float32 n=1024 B=64 29 us per frame with 16 rows, 35 with 32; 64 rows were never faster).
  int NT = B > 16 ? 2 : 1;
  if (NT > 1 && (long long)(n / 16) * ((B + 16 * NT - 1) / (16 * NT)) < device_info().cus) NT = 1;
  auto record = [&](LaunchSink& sink) -> int {
    const dim3 pw_grid((unsigned)((x.bn + 255) / 256)), pw_block(256);
    const dim3 mm_grid((unsigned)((n / 16) * ((B + 16 * NT - 1) / (16 * NT)))), mm_block(kWgThreads);
    const bool bf = dtype == RTN_DTYPE_BF16;
    long long t_done = -1;  // frame whose DX still has to go through the GEMM
    for (long long t = end;; t -= step) {
      const bool more = step > 0 ? t >= first : t <= first;
      const bool right = more && (step > 0 ? (t - step >= first) : (t - step <= first));
      const long long prev_t = right ? t - step : -1;
      const long long tt = more ? t : -1;
      int rc2 = RTN_OK;
      if (mfma) {
        void (*k)(Lstm2BwdParams, long long, long long, long long) =
            bf ? (NT == 2 ? &k_bwd_step<__bf16, 2> : &k_bwd_step<__bf16, 1>) : (NT == 2 ? &k_bwd_step<float, 2> : &k_bwd_step<float, 1>);
        rc2 = enqueue(sink, k, mm_grid, mm_block, 0, p, t_done, tt, prev_t);
      } else if (more) {
        rc2 = enqueue(sink, bf ? &k_bwd_pointwise<__bf16> : &k_bwd_pointwise<float>, pw_grid, pw_block, 0, p, t, prev_t);
        if (rc2 == RTN_OK)
          rc2 = enqueue(sink, bf ? &k_bwd_gemm_dy_generic<__bf16> : &k_bwd_gemm_dy_generic<float>, pw_grid, pw_block, 0, p, t);
      }
      if (rc2 != RTN_OK) return rc2;
      if (!more) break;
      t_done = t;
    }
    return RTN_OK;
  };
  if (x.capturing || env_long("RTN_LSTM2_BWD_NO_GRAPH", 0)) {
    LaunchSink sink;
    sink.stream = stream;
    return record(sink);
  }
  std::string key("bwd");
  int dev = 0;
  RTN_HIP(hipGetDevice(&dev));
  Lstm2BwdParams shape = p;  // p was zeroed before it was filled in
  shape.W = shape.H = shape.DY = shape.Wpk = nullptr;
  shape.c0 = shape.mask = shape.C = nullptr;
  shape.DX = shape.dx0 = nullptr;
  shape.dyw = shape.Dc0 = nullptr;
  key.append(reinterpret_cast<const char*>(&shape), sizeof(shape));
  key_append(&key, (int)(p.Wpk != nullptr));
  key_append(&key, dtype); key_append(&key, (int)x.calls[0].start); key_append(&key, step); key_append(&key, dev);
  key_append(&key, (int)mfma); key_append(&key, NT);
  return replay_graph(key, &p, sizeof(p), stream, record);
}

// DW = sum over consecutive visited frames Y[t - step]^T * DX[t]  (returnn/native_op.py:1433-1452), then += y0^T * dx0
// (:1456-1460), in rocBLAS; where the recurrence ran per frame, Dy0 from its float32 working copy.
int bwd_weight_gradients(const BwdCtx& x, rocblas_handle blas, const std::vector<BwdJob>& jobs, bool persistent) {
  const int n = x.n, B = x.B;
  const dim3 fill_grid(256), fill_block(256);
  int rc = RTN_OK;
  for (int k = 0; k < x.count; ++k) {
    const rtn_lstm2_bwd_call& c = x.calls[k];
    const BwdJob& j = jobs[(size_t)k];
    const int step = c.step;
    const unsigned char* Yb = (const unsigned char*)c.Y;
    const unsigned char* DXb = (const unsigned char*)c.DX;
    if (j.num_steps > 1) {
      if (j.abs_step == 1) {
        const long long lo = std::min(j.first, j.end);
        rc = dw_accumulate(blas, Yb + (size_t)(lo + std::max(0, -step)) * B * j.ldY * x.es,
                           DXb + (size_t)(lo + std::max(0, step)) * B * j.p.ldDX * x.es, c.DW, (j.num_steps - 1) * B, n, x.dtype, j.ldY, j.p.ldDX);
        if (rc != RTN_OK) return rc;
      } else {
        for (long long t = j.end - step; step > 0 ? t >= j.first : t <= j.first; t -= step) {
          rc = dw_accumulate(blas, Yb + (size_t)t * B * j.ldY * x.es, DXb + (size_t)(t + step) * B * j.p.ldDX * x.es, c.DW, B, n, x.dtype, j.ldY,
                             j.p.ldDX);
          if (rc != RTN_OK) return rc;
        }
      }
    }
    rc = dw_accumulate(blas, c.y0, j.p.dx0, c.DW, B, n, x.dtype);
    if (rc != RTN_OK) return rc;
    if (!persistent) {
      if (x.dtype == RTN_DTYPE_BF16)
        hipLaunchKernelGGL(k_convert_from_f32<__bf16>, fill_grid, fill_block, 0, x.stream, j.p.dyw, c.Dy0, x.bn);
      else
        hipLaunchKernelGGL(k_convert_from_f32<float>, fill_grid, fill_block, 0, x.stream, j.p.dyw, c.Dy0, x.bn);
      RTN_HIP(hipGetLastError());
    }
  }
  return RTN_OK;
}

// `count` gradient calls of one shape.  With the persistent kernel and count <= kMaxBwdMulti all of them share one
// launch (16-row batch groups when 8-row groups of all problems would not find a CU each); otherwise they are enqueued
// one after the other.
int bwd_calls(const rtn_lstm2_bwd_call* calls, int count, int64_t T, int32_t B, int32_t n, int32_t dtype, void* workspace,
              size_t workspace_bytes, void* hip_stream, int op_flags, size_t ws_stride) {
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (count < 0 || (count > 0 && !calls)) return fail(RTN_ERR_ARG, "NativeLstm2 backward: bad call list");
  BwdCtx x;
  x.calls = calls; x.count = count; x.T = T; x.B = B; x.n = n; x.dtype = dtype; x.op_flags = op_flags;
  x.stream = (hipStream_t)hip_stream;
  x.es = esize(dtype);
  x.bn = (long long)B * n;
  hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
  if (x.stream) RTN_HIP(hipStreamIsCapturing(x.stream, &cap_status));
  // Under stream capture everything is recorded into the caller's graph: the persistent kernel as a kernel node of its
  // own (launch_coresident) or one launch per frame, and the rocBLAS calls of the weight gradient (the library's rocBLAS
  // handle must exist already: run the op once outside the capture first, as for any library that sets itself up on
  // first use).
  x.capturing = cap_status != hipStreamCaptureStatusNone;
  if (!x.capturing && T > 0 && x.bn > 0 && (rc = probe_xcds(x.stream)) != RTN_OK) return rc;
  if ((rc = bwd_check_and_clear(x)) != RTN_OK) return rc;
  if (T == 0 || x.bn == 0 || count == 0) return RTN_OK;
  const int np = padded_width(n);
  if (np != n) return bwd_padded(x, np, workspace, workspace_bytes);

  const BwdLayout lay = bwd_layout(B, n, dtype);
  const size_t stride = ws_stride ? ws_stride : lay.total;  // distance between the calls' workspaces
  if (stride < lay.total) return fail(RTN_ERR_WORKSPACE, "NativeLstm2 backward: internal: workspace slice %zu < layout %zu", stride, lay.total);
  if (!workspace || workspace_bytes < stride * (size_t)(count - 1) + lay.total)
    return fail(RTN_ERR_WORKSPACE, "NativeLstm2 backward: workspace of %zu bytes needed, got %zu", stride * (size_t)(count - 1) + lay.total,
                workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "NativeLstm2 backward: workspace must be 16-byte aligned");
  rocblas_handle blas = nullptr;
  rc = blas_handle(&blas);
  if (rc != RTN_OK) return rc;
  if (rocblas_set_stream(blas, x.stream) != rocblas_status_success) return fail(RTN_ERR_HIP, "NativeLstm2 backward: rocblas_set_stream failed");
  const bool mfma = (n % 16) == 0 && !env_long("RTN_LSTM2_FORCE_GENERIC", 0);

  BwdChoice ch;
  const long bwd_kernel = env_long("RTN_LSTM2_BWD_KERNEL", 0);  // 0 auto, 1 per-frame launches, 2 persistent
  const int KM = dtype == RTN_DTYPE_BF16 ? 32 : 16;
  if (mfma && (4 * n) % KM == 0 && bwd_kernel != 1 && (!x.capturing || capture_keeps_persistent()) && device_info().cooperative && count <= kMaxBwdMulti)
    if ((rc = choose_bwd_kernel(x, &ch)) != RTN_OK) return rc;
  if (!ch.kernel && count > 1) {
    // no joint launch: one call after the other, each with its own slice of the workspace
    for (int k = 0; k < count; ++k) {
      rc = bwd_calls(calls + k, 1, T, B, n, dtype, (unsigned char*)workspace + (size_t)k * stride, lay.total, hip_stream, op_flags);
      if (rc != RTN_OK) return rc;
    }
    return RTN_OK;
  }
  if (bwd_kernel == 2 && !ch.kernel)
    return fail(RTN_ERR_UNSUPPORTED, "NativeLstm2 backward: the persistent kernel cannot run T=%lld B=%d n=%d", (long long)T, B, n);
  {
    const int bgroups = (B + ch.rows_per_group - 1) / ch.rows_per_group;
    char buf[256];
    if (ch.kernel)
      snprintf(buf, sizeof(buf), "kernel=%s problems=%d rows_per_group=%d groups=%d tiles=%d waves=%d wgs_per_group=%d launches=%d",
               ch.local ? "bwd_regw_xcd" : "bwd_regw", count, ch.rows_per_group, bgroups, ch.tiles, ch.waves, n / (16 * ch.tiles),
               (bgroups + ch.groups_per_launch - 1) / std::max(ch.groups_per_launch, 1));
    else
      snprintf(buf, sizeof(buf), "kernel=%s problems=%d launches_per_frame=%d", mfma ? "bwd_step" : "bwd_generic", count, mfma ? 1 : 2);
    g_bwd_plan_text = buf;
  }

  std::vector<BwdJob> jobs;
  if ((rc = bwd_prepare_jobs(x, ch, lay, workspace, stride, &jobs)) != RTN_OK) return rc;
  rc = ch.kernel ? bwd_launch_persistent(x, ch, lay, jobs) : bwd_launch_per_frame(x, mfma, lay, jobs[0]);  // (per frame: count == 1)
  if (rc != RTN_OK) return rc;
  return bwd_weight_gradients(x, blas, jobs, ch.kernel != nullptr);
}

}  // namespace

int rtn_native_lstm2_bwd(const void* W, const void* y0, const float* c0, const float* i, int32_t start, int32_t step,
                         const void* Y, const float* C, const void* H, const void* DY, const float* Dd, void* DX, float* DW,
                         void* Dy0, float* Dc0, int64_t T, int32_t B, int32_t n, int32_t dtype, void* workspace,
                         size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  const rtn_lstm2_bwd_call call = {W, y0, c0, i, start, step, Y, C, H, DY, Dd, DX, DW, Dy0, Dc0};
  return bwd_calls(&call, 1, T, B, n, dtype, workspace, workspace_bytes, hip_stream);
}

size_t rtn_lstm_generic_base_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype) {
  const size_t bwd = rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dtype);
  if (bwd == 0) return 0;
  // gradient workspace | zero initial output [B,n] | error of the initial output [B,n] (the op has neither)
  return align_up(bwd, 256) + 2 * align_up((size_t)B * n * esize(dtype), 256);
}

int rtn_lstm_generic_base_bwd(const void* V_h, const float* c, const float* i, const void* Y, const void* H, const void* DY,
                              const float* Dd, void* DZ, float* DV_h, float* Dc, int64_t T, int32_t B, int32_t n, int32_t dtype,
                              void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (T == 0) return fail(RTN_ERR_SHAPE, "LstmGenericBase gradient: needs T > 0");  // returnn/native_op.py:547
  const size_t need = rtn_lstm_generic_base_bwd_workspace_bytes(T, B, n, dtype);
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "LstmGenericBase gradient: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "LstmGenericBase gradient: workspace must be 16-byte aligned");
  const size_t bwd = align_up(rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dtype), 256);
  const size_t state_bytes = align_up((size_t)B * n * esize(dtype), 256);
  unsigned char* ws = (unsigned char*)workspace;
  void* y0 = ws + bwd;
  void* Dy0 = ws + bwd + state_bytes;
  if ((long long)B * n > 0) {
    hipLaunchKernelGGL(k_fill_u32, dim3(64), dim3(256), 0, (hipStream_t)hip_stream, (unsigned*)y0, 0u, (long long)(state_bytes / 4));
    RTN_HIP(hipGetLastError());
  }
  // the cell states are the first block of H (kOpH0IsCell); the C argument is not read then
  const rtn_lstm2_bwd_call call = {V_h, y0, c, i, 0, 1, Y, (const float*)H, H, DY, Dd, DZ, DV_h, Dy0, Dc};
  return bwd_calls(&call, 1, T, B, n, dtype, workspace, bwd, hip_stream, kOpNoCarry | kOpH0IsCell);
}

namespace {
constexpr int kColumnSumParts = 64;
struct LowMemBwdLayout {
  size_t bwd = 0, H = 0, DI = 0, partial = 0, total = 0;
};
void low_mem_bwd_layout(int64_t T, int B, int n, int dtype, LowMemBwdLayout* out) {
  LowMemBwdLayout l;
  l.bwd = 0;
  size_t off = align_up(rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dtype), 256);
  const size_t frames = align_up((size_t)T * B * 4 * n * esize(dtype), 256);
  l.H = off;
  off += frames;
  l.DI = off;
  off += frames;
  l.partial = off;
  off += align_up((size_t)kColumnSumParts * 4 * n * 4, 256);
  l.total = off;
  *out = l;
}
}  // namespace

size_t rtn_lstm_low_mem_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype) {
  (void)n_in;
  if (check_dims(T, B, n, dtype) != RTN_OK) return 0;
  if (rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dtype) == 0) return 0;
  // gradient workspace of the recurrence | gates [T,B,4n] | their derivatives [T,B,4n] | partial column sums
  LowMemBwdLayout l;
  low_mem_bwd_layout(T, B, n, dtype, &l);
  return l.total;
}

int rtn_lstm_low_mem_bwd(const void* X, const void* W, const void* b, const void* y0, const float* c0, const float* i, int32_t start,
                         int32_t step, const void* Y, const float* C, const void* DY, const float* Dd, void* DX, float* DW, float* Db,
                         void* Dh, float* Dc, int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype, void* workspace,
                         size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if (n_in < 0) return fail(RTN_ERR_SHAPE, "LstmLowMem gradient: negative input dimension %d", n_in);
  if (T == 0) return fail(RTN_ERR_SHAPE, "LstmLowMem gradient: needs T > 0");  // returnn/native_op.py:953
  if (start < 0 || start >= T) return fail(RTN_ERR_RANGE, "LstmLowMem gradient: need 0 <= start < T, got start=%d, T=%lld", start, (long long)T);
  if (step == 0) return fail(RTN_ERR_RANGE, "LstmLowMem gradient: step must not be 0");
  // The reference's loop walks back from frame T-1 (step > 0) or up from frame `start` (step < 0) whatever the stride
  // (:957-964); those are the frames its forward pass visited only if the stride divides the distance between the two
  // ends.  Otherwise it would read outputs of frames that were never computed: refused.
  const long long first = step > 0 ? start : T - start - 1, far_end = step > 0 ? T - 1 : start, astep = step > 0 ? step : -(long long)step;
  if (step < 0 && first < far_end)
    return fail(RTN_ERR_RANGE, "LstmLowMem gradient: start=%d with a negative step visits no frame of T=%lld", start, (long long)T);
  if ((step > 0 ? far_end - first : first - far_end) % astep != 0)
    return fail(RTN_ERR_RANGE, "LstmLowMem gradient: the stride %d does not divide the distance between frame %lld and frame %lld; the reference's gradient loop would visit frames its forward pass did not", step, first, far_end);
  const long long num_steps = (step > 0 ? far_end - first : first - far_end) / astep + 1;
  hipStream_t stream = (hipStream_t)hip_stream;
  const size_t need = rtn_lstm_low_mem_bwd_workspace_bytes(T, B, n_in, n, dtype);
  const long long bn = (long long)B * n, rows = (long long)T * B;
  const size_t es = esize(dtype);
  if (bn == 0) {
    if (n_in > 0 && rows > 0) {
      if (!DX) return fail(RTN_ERR_ARG, "LstmLowMem gradient: DX must not be null");
      hipLaunchKernelGGL(k_fill_u32, dim3(256), dim3(256), 0, stream, (unsigned*)DX, 0u, (long long)(((size_t)rows * n_in * es + 3) / 4));
      RTN_HIP(hipGetLastError());
    }
    return RTN_OK;
  }
  if (!workspace || workspace_bytes < need)
    return fail(RTN_ERR_WORKSPACE, "LstmLowMem gradient: workspace of %zu bytes needed, got %zu", need, workspace ? workspace_bytes : (size_t)0);
  if (!aligned16(workspace)) return fail(RTN_ERR_ARG, "LstmLowMem gradient: workspace must be 16-byte aligned");
  {
    const void* ptrs[] = {X, W, b, y0, c0, i, Y, C, DY, Dd, DX, DW, Db, Dh, Dc};
    const char* names[] = {"X", "W", "b", "y0", "c0", "i", "Y", "C", "DY", "Dd", "DX", "DW", "Db", "Dh", "Dc"};
    for (int q = 0; q < 15; ++q) {
      if (!ptrs[q] && !((q == 0 || q == 10) && n_in == 0)) return fail(RTN_ERR_ARG, "LstmLowMem gradient: %s must not be null", names[q]);
      if (q != 5 && ptrs[q] && !aligned16(ptrs[q])) return fail(RTN_ERR_ARG, "LstmLowMem gradient: %s must be 16-byte aligned", names[q]);
    }
  }
  LowMemBwdLayout L;
  low_mem_bwd_layout(T, B, n, dtype, &L);
  unsigned char* ws = (unsigned char*)workspace;
  void* H = ws + L.H;
  void* DI = ws + L.DI;
  float* partial = (float*)(ws + L.partial);
  const unsigned char* W_rec = (const unsigned char*)W + (size_t)n_in * 4 * n * es;  // rows n_in.. of W: the recurrent part
  float* DW_rec = DW + (size_t)n_in * 4 * n;
  rocblas_handle blas = nullptr;
  rc = blas_handle(&blas);
  if (rc != RTN_OK) return rc;
  if (rocblas_set_stream(blas, stream) != rocblas_status_success) return fail(RTN_ERR_HIP, "LstmLowMem gradient: rocblas_set_stream failed");
  const rocblas_datatype ty = dtype == RTN_DTYPE_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f32_r;
  const int n4 = 4 * n;
  const unsigned char* Yb = (const unsigned char*)Y;
  unsigned char* Hb = (unsigned char*)H;
  const size_t y_frame = (size_t)bn * es, h_frame = (size_t)bn * 4 * es;

  // 1. The pre-activations of every frame again (:966-979): [X[t], Y[t-step] or y0] W.  The outputs are all known, so
  //    this is no recurrence: one GEMM over all frames for the input part, one over all visited frames but the first
  //    for the recurrent part (per frame if the stride is not 1), one for the first frame with y0.
  if (n_in > 0) {
    rc = gemm_row_major(blas, false, false, rows, n4, n_in, X, n_in, W, n4, ty, 0.f, H, n4, ty);
    if (rc != RTN_OK) return rc;
  } else {
    hipLaunchKernelGGL(k_fill_u32, dim3(1024), dim3(256), 0, stream, (unsigned*)H, 0u, (long long)(((size_t)rows * n4 * es + 3) / 4));
    RTN_HIP(hipGetLastError());
  }
  if (num_steps > 1) {
    if (astep == 1) {
      const long long lo = std::min(first, first + (num_steps - 1) * step);
      // step +1: frames lo+1.. take Y[lo..]; step -1: frames lo.. take Y[lo+1..]
      rc = gemm_row_major(blas, false, false, (num_steps - 1) * B, n4, n, Yb + (size_t)(lo + (step < 0 ? 1 : 0)) * y_frame, n, W_rec, n4, ty, 1.f,
                          Hb + (size_t)(lo + (step > 0 ? 1 : 0)) * h_frame, n4, ty);
      if (rc != RTN_OK) return rc;
    } else {
      for (long long s = 1; s < num_steps; ++s) {
        const long long t = first + s * step;
        rc = gemm_row_major(blas, false, false, B, n4, n, Yb + (size_t)(t - step) * y_frame, n, W_rec, n4, ty, 1.f, Hb + (size_t)t * h_frame, n4, ty);
        if (rc != RTN_OK) return rc;
      }
    }
  }
  rc = gemm_row_major(blas, false, false, B, n4, n, y0, n, W_rec, n4, ty, 1.f, Hb + (size_t)first * h_frame, n4, ty);
  if (rc != RTN_OK) return rc;
  {
    const long long total = rows * n4;
    const dim3 grid((unsigned)std::min<long long>((total + 255) / 256, 65535)), block(256);
    if (dtype == RTN_DTYPE_BF16)
      hipLaunchKernelGGL(k_low_mem_gates<__bf16>, grid, block, 0, stream, H, b, rows, n);
    else
      hipLaunchKernelGGL(k_low_mem_gates<float>, grid, block, 0, stream, H, b, rows, n);
    RTN_HIP(hipGetLastError());
  }
  // 2. The recurrence of the errors (:981-1017 without the two large products): the gradient kernels of NativeLstm2 on
  //    the recurrent rows of W, with this op's variations.  Gives the derivatives of the pre-activations (DI), the
  //    recurrent rows of DW, Dh and Dc.
  const rtn_lstm2_bwd_call call = {W_rec, y0, c0, i, start, step, Y, C, H, DY, Dd, DI, DW_rec, Dh, Dc};
  rc = bwd_calls(&call, 1, T, B, n, dtype, workspace, L.H, hip_stream, kOpNoCarry | kOpRawDh | kOpEndAtStart);
  if (rc != RTN_OK) return rc;
  // 3. What the reference accumulates frame by frame, as products over all frames at once (DI is 0 in frames that were not
  //    visited): DX = DI W_x^T (:1001-1007, :1016), the input rows of DW = X^T DI (:1009-1014), Db = column sums of DI (:704-707).
  if (n_in > 0) {
    rc = gemm_row_major(blas, false, true, rows, n_in, n4, DI, n4, W, n4, ty, 0.f, DX, n_in, ty);
    if (rc != RTN_OK) return rc;
    rc = gemm_row_major(blas, true, false, n_in, n4, rows, X, n_in, DI, n4, ty, 0.f, DW, n4, rocblas_datatype_f32_r);
    if (rc != RTN_OK) return rc;
  }
  {
    const dim3 block(256), grid1((unsigned)((n4 + 255) / 256), kColumnSumParts), grid2((unsigned)((n4 + 255) / 256));
    if (dtype == RTN_DTYPE_BF16)
      hipLaunchKernelGGL(k_column_partial_sums<__bf16>, grid1, block, 0, stream, DI, partial, rows, n4);
    else
      hipLaunchKernelGGL(k_column_partial_sums<float>, grid1, block, 0, stream, DI, partial, rows, n4);
    hipLaunchKernelGGL(k_column_final_sums, grid2, block, 0, stream, partial, Db, kColumnSumParts, n4);
    RTN_HIP(hipGetLastError());
  }
  return RTN_OK;
}

size_t rtn_native_lstm2_bwd_multi_workspace_bytes(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype) {
  if (count < 0) return 0;
  return (size_t)count * rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dtype);
}

int rtn_native_lstm2_bwd_multi(const rtn_lstm2_bwd_call* calls, int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype,
                               void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_last_error.clear();
  return bwd_calls(calls, count, T, B, n, dtype, workspace, workspace_bytes, hip_stream);
}

#ifdef RTN_LSTM2_TRACE
// Instrumented builds only: the per-workgroup phase times of the last persistent gradient launch.
__attribute__((visibility("default"))) int rtn_debug_bwd_trace(unsigned long long* out, int workgroups) {
  if (workgroups > 1024) workgroups = 1024;
  RTN_HIP(hipDeviceSynchronize());
  RTN_HIP(hipMemcpyFromSymbol(out, HIP_SYMBOL(rtn::g_bwd_trace), (size_t)workgroups * 8 * sizeof(unsigned long long)));
  return RTN_OK;
}
#endif

int rtn_native_lstm2_fwd_status(const void* workspace, void* hip_stream) {
  g_last_error.clear();
  if (!workspace) return fail(RTN_ERR_ARG, "NativeLstm2: workspace must not be null");
  unsigned status = 0;
  hipStream_t stream = (hipStream_t)hip_stream;
  RTN_HIP(hipMemcpyAsync(&status, workspace, sizeof(status), hipMemcpyDeviceToHost, stream));
  RTN_HIP(hipStreamSynchronize(stream));
  if (status == 2)
    return fail(RTN_ERR_ABORTED, "NativeLstm2: the last run on this workspace was a measurement aid (exchange probe or no-wait timing); it computes no outputs");
  if (status != 0) return fail(RTN_ERR_ABORTED, "NativeLstm2: a bounded wait in the persistent kernel expired; outputs are invalid");
  return RTN_OK;
}

int rtn_native_lstm2_last_output(const void* Y, const void* y0, const float* i, int32_t start, int32_t step, void* out,
                                 int64_t T, int32_t B, int32_t n, int32_t dtype, int64_t ldY, void* hip_stream) {
  g_last_error.clear();
  int rc = check_dims(T, B, n, dtype);
  if (rc != RTN_OK) return rc;
  if ((long long)B * n == 0) return RTN_OK;
  if (!y0 || !out) return fail(RTN_ERR_ARG, "NativeLstm2: y0 and out must not be null");
  if (ldY != 0 && ldY < n) return fail(RTN_ERR_ARG, "NativeLstm2: row pitch ldY=%lld is below the row length %d", (long long)ldY, n);
  const long long ld = ldY ? ldY : n;
  int first = 0, nsteps = 0;
  if (T > 0) {
    if (start < 0 || start >= T) return fail(RTN_ERR_RANGE, "NativeLstm2: need 0 <= start < T, got start=%d, T=%lld", start, (long long)T);
    if (step == 0) return fail(RTN_ERR_RANGE, "NativeLstm2: step must not be 0");
    if (!Y || !i) return fail(RTN_ERR_ARG, "NativeLstm2: Y and i must not be null");
    if (step > 0) {
      first = start;
      nsteps = (int)((T - 1 - start) / step + 1);
    } else {
      first = (int)(T - start - 1);
      nsteps = (int)(first / (-(long long)step) + 1);
    }
  }
  hipStream_t stream = (hipStream_t)hip_stream;
  if (dtype == RTN_DTYPE_BF16)
    hipLaunchKernelGGL(k_last_output<__bf16>, dim3(B), dim3(256), 0, stream, Y, y0, i, out, (long long)T, B, n, first, step, nsteps, ld);
  else
    hipLaunchKernelGGL(k_last_output<float>, dim3(B), dim3(256), 0, stream, Y, y0, i, out, (long long)T, B, n, first, step, nsteps, ld);
  RTN_HIP(hipGetLastError());
  return RTN_OK;
}

}  // extern "C"
