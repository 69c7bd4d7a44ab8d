// C ABI of the engine (include/crl.h): owns the device buffers, validates
// arguments on the host and launches the gfx950 kernels of crl_kernels.h.
// There is no CPU fallback anywhere in this file.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "../../include/crl.h"
#include "crl_host.h"
#include "crl_kernels.h"
#include "crl_persist.h"

namespace {

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  return crl::fail_with(code, buf);
}

#define HIP_TRY(expr)                                                                   \
  do {                                                                                  \
    hipError_t _e = (expr);                                                             \
    if (_e != hipSuccess)                                                               \
      return fail(_e == hipErrorOutOfMemory ? CRL_E_ALLOC : CRL_E_DEVICE, "%s: %s (%s:%d)", \
                  #expr, hipGetErrorString(_e), __FILE__, __LINE__);                    \
  } while (0)

// Runs the body of an entry point that allocates host memory or starts threads:
// nothing may throw across the C ABI.
template <class F>
int guarded(F&& body) {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return fail(CRL_E_ALLOC, "host allocation failed");
  } catch (const std::exception& x) {
    return fail(CRL_E_DEVICE, "%s", x.what());
  } catch (...) {
    return fail(CRL_E_DEVICE, "unknown failure");
  }
}

template <class T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  hipError_t alloc(size_t count) {
    release();
    if (count == 0) return hipSuccess;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&p), count * sizeof(T));
    if (e == hipSuccess) n = count;
    else p = nullptr;
    return e;
  }
  hipError_t ensure(size_t count) { return count <= n ? hipSuccess : alloc(count); }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    n = 0;
  }
  ~DevBuf() { release(); }
  DevBuf() = default;
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
};

// Scratch of crl_run_fused_noalloc: one array per GPU, part of the loaded code
// object, so the entry point never allocates.  Layout: 4 KB of counters (the ticket
// counters), then 10 MB for what the workgroups of a shared-table step exchange: the
// hand-off cells of the ordered reduction, or all exchange buffers of the one-launch
// kernel.  The array's name
// is a host-side stand-in, not a device address: host code only ever uses the
// address hipGetSymbolAddress returned for the device at hand.
constexpr size_t kScratchTicketBytes = 4096;
constexpr size_t kScratchExchangeBytes = (size_t)10 << 20;
constexpr size_t kScratchBytes = kScratchTicketBytes + kScratchExchangeBytes;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

// Address of `device`'s copy of the scratch array; looked up once per device, with
// that device current.  Called from crl_create, so that crl_run_fused_noalloc
// finds it there.
int scratch_of_device(int device, unsigned char** out) {
  if (device < 0 || device >= kMaxDevices) return fail(CRL_E_ARG, "device %d: at most %d devices", device, kMaxDevices);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[device]) {
    HIP_TRY(hipSetDevice(device));
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(CRL_E_DEVICE, "hipGetSymbolAddress returned no address for the scratch array");
    g_scratch_ptr[device] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[device];
  return CRL_OK;
}

}  // namespace

struct crl_engine {
  crl_config cfg{};
  int device = 0;
  hipStream_t stream = nullptr;
  int N = 0, W = 0, H = 0, A = 0;
  size_t S = 0, K = 0;
  int n_maps = 0, n_tables = 0, map_words = 0;
  int mv_words = 0;  // words of move codes per map; 0: no move codes are kept
  uint64_t t = 0;
  long resident_envs = 0;  // 0 = automatic
  int fused_variant = 0;   // 0 = automatic, 1 = plain, 2 = hybrid (when it fits)
  DevBuf<unsigned> ticket;
  DevBuf<unsigned> split;  // the engine's own copy of the last launch's ticket counters (crl_get_fused_split)
  bool hybrid_opt_in = false;
  // the scratch the call in progress works with: the engine's own allocations
  // (crl_run_fused, crl_update, crl_td_update) or the device's static array
  // (crl_run_fused_noalloc)
  bool no_alloc = false;
  unsigned char* static_scratch = nullptr;
  unsigned* tk = nullptr;  // ticket counters {next ticket, envs on HBM tables, envs on LDS tables}
  bool split_valid = false;  // the last fused launch drew tickets
  unsigned long long* ho = nullptr;  // hand-off cells of the ordered reduction
  // one-launch shared-table kernel: what its workgroups exchange (the tagged views of
  // the table's cells, raw samples, hand-off cells), the engine's own give-up word
  // followed by the phase clocks, and whether a launch has not been checked for
  // having given up yet
  DevBuf<unsigned long long> pbuf;
  DevBuf<unsigned long long> pdiag;  // [0] give-up word, [1..16] phase clocks; allocated at crl_create
  bool persist_unchecked = false;
  bool persist_failed = false;   // a launch gave up: state and table are not valid until they are set again
  bool persist_refused = false;  // the device refused the co-resident launch once: not tried again
  bool persist_clocks = false;   // run the instantiation that keeps phase clocks
  int persist_spin_limit = crl::kPersistSpinLimit;  // polls a thread waits for its peers before it gives up

  DevBuf<int32_t> s, ep_step, episode, start, act;
  DevBuf<float> reward;
  DevBuf<uint8_t> done, action;
  DevBuf<uint32_t> map;
  DevBuf<uint32_t> moves;  // move codes derived from map, for the folded fused loop
  DevBuf<float> cell_reward;
  DevBuf<float> Q;
  DevBuf<float> eps_tab;
  int eps_len = 1;
  // episode statistics (allocated when cfg.track_returns)
  DevBuf<float> ret_acc, ret_last, ret_sum;
  DevBuf<int32_t> len_last, len_sum;
  // transition of the last crl_step
  DevBuf<int32_t> tr_s, tr_a, tr_s2;
  DevBuf<float> tr_r;
  DevBuf<uint8_t> tr_done;
  bool have_transition = false, have_actions = false;
  // (key, delta) scratch of the ordered reduction, and the block sums its
  // first pass hands to the key owners
  DevBuf<int32_t> key;
  DevBuf<float> delta;
  DevBuf<unsigned long long> handoff;
  bool lds_opt_in = false;
  // scratch of crl_td_update
  DevBuf<int32_t> b_s, b_a, b_s2;
  DevBuf<float> b_r;
  DevBuf<uint8_t> b_done;
  // trace
  DevBuf<int32_t> trace_s;
  DevBuf<uint8_t> trace_a, trace_d;
  DevBuf<float> trace_r;
  int trace_n = 0, trace_cap = 0, trace_cursor = 0;
  // supplied exploration stream
  DevBuf<float> u_sup;
  DevBuf<int32_t> a_sup;
  uint64_t sup_t0 = 0;
  int sup_n = 0;

  crl::Rules rules() const {
    crl::Rules R{};
    R.W = W;
    R.H = H;
    R.A = A;
    R.goal_mode = cfg.goal_mode;
    R.reward_flags = cfg.reward_flags;
    R.auto_reset = cfg.auto_reset;
    R.episode_len = cfg.episode_len;
    R.max_mode = cfg.max_mode;
    R.eps_mode = cfg.eps_mode;
    R.eps_len = eps_len;
    R.max_episodes = cfg.max_episodes;
    R.lr = cfg.lr;
    R.gamma = cfg.gamma;
    R.step_reward = cfg.step_reward;
    R.goal_reward = cfg.goal_reward;
    R.trap_reward = cfg.trap_reward;
    R.eps0 = cfg.eps0;
    R.seed = cfg.seed;
    return R;
  }
  crl::Ptrs ptrs() const {
    crl::Ptrs P{};
    P.s = s.p;
    P.ep_step = ep_step.p;
    P.episode = episode.p;
    P.start = start.p;
    P.reward = reward.p;
    P.done = done.p;
    P.action = action.p;
    P.map = map.p;
    P.moves = moves.p;
    P.cell_reward = (cfg.reward_flags & CRL_REWARD_CELLS) ? cell_reward.p : nullptr;
    P.Q = Q.p;
    P.eps_tab = eps_tab.p;
    P.u_sup = sup_n > 0 ? u_sup.p : nullptr;
    P.a_sup = a_sup.p;
    P.sup_t0 = sup_t0;
    P.sup_n = sup_n;
    P.tr_s = trace_s.p;
    P.tr_a = trace_a.p;
    P.tr_r = trace_r.p;
    P.tr_d = trace_d.p;
    P.trace_n = trace_n;
    P.trace_cursor = trace_cursor;
    P.trace_cap = trace_cap;
    P.ret_acc = ret_acc.p;
    P.ret_last = ret_last.p;
    P.ret_sum = ret_sum.p;
    P.len_last = len_last.p;
    P.len_sum = len_sum.p;
    P.N = N;
    P.map_words = map_words;
    P.mv_words = mv_words;
    P.map_shared = cfg.map_mode == CRL_MAP_SHARED;
    P.table_shared = cfg.table_mode == CRL_TABLE_SHARED;
    P.S = S;
    return P;
  }
  crl::Transition transition() const {
    crl::Transition T{};
    T.s = tr_s.p;
    T.a = tr_a.p;
    T.r = tr_r.p;
    T.s2 = tr_s2.p;
    T.done = tr_done.p;
    return T;
  }
};

namespace {

constexpr int kLdsMapLimitBytes = 64 * 1024;
// Table bytes to keep in flight at once: three quarters of the MI355X Infinity
// Cache (256 MB).  Measured on 4 KB tables (table waves alone): 128 MB in flight 5.9e10 env-steps/s,
// 192 MB 6.3e10, 256 MB 5.2e10, 384 MB 3.9e10.
constexpr size_t kTableBytesInFlight = (size_t)192 << 20;
constexpr int kComputeUnits = 256;
constexpr long kMinEnvsInFlight = kComputeUnits * 3L * 64;  // three waves per compute unit
constexpr int kInFlightMinSteps = 16;  // shorter launches: 4 steps 6.1e9 -> 6.9e9 with all envs in flight

// launch geometry of the fused per-env kernel
struct FusedPlan {
  int map_kind;  // 0 per-env LDS, 1 shared LDS, 2 global
  int block, grid;
  size_t lds;
  const char* name;
  bool tickets;    // per-env maps in LDS: waves draw env ranges from a ticket counter
  bool hybrid;     // ... whose last wave per workgroup steps envs whose tables it holds in LDS
  bool fast;       // the folded loop for the common configuration
  bool moves;      // ... whose table waves read pre-built move codes from LDS
  bool fixed;      // tickets dealt by position, round after round: no counter
  bool pair;       // per-env kernel: two lanes per env
  int pair_envs;   // ticket kernel: envs per thin table wave (32, 16, 8), 0: 64-env waves
  bool rich;       // ticket kernel: the folded loop's variant with per-cell rewards / per-episode epsilon
  int tab_stride;  // floats between two tables in LDS
};

constexpr size_t kLdsPerWorkgroup = 160 * 1024;  // gfx950
// static LDS of kernels that call the workgroup-wide "or" (the device library keeps a few
// words there), rounded up: their dynamic LDS can be at most the rest
constexpr size_t kStaticLdsReserve = 1024;

// Launches shorter than this do not repay moving whole tables into LDS and back
// (1M envs of config 4, steps per launch -> env-steps/s, plain / hybrid:
// 32: 2.4e10 / 2.1e10, 48: 2.8e10 / 2.75e10, 64: 3.0e10 / 3.3e10, 100: 3.6e10 / 4.2e10).
constexpr int kHybridMinSteps = 64;
constexpr int kStagedMovesMinSteps = 128;

FusedPlan plan_fused(const crl_engine* e, int n_steps) {
  FusedPlan p{};
  // small batches spread over more compute units with one-wave blocks
  p.block = e->N >= 256 * 512 ? 256 : 64;
  if (e->cfg.map_mode == CRL_MAP_SHARED) {
    if ((size_t)e->mv_words * 4 <= (size_t)kLdsMapLimitBytes) {
      p.map_kind = 1;
      p.lds = (size_t)e->mv_words * 4;  // the shared map's move codes
    } else {
      p.map_kind = 2;
    }
  } else {
    if ((size_t)e->map_words * 4 * 64 <= (size_t)kLdsMapLimitBytes) {
      p.map_kind = 0;
      while ((size_t)e->map_words * 4 * p.block > (size_t)kLdsMapLimitBytes) p.block /= 2;
      p.lds = (size_t)e->map_words * 4 * p.block;
    } else {
      p.map_kind = 2;
    }
  }
  // Envs live on the chip at once.  A worker steps its envs for all n steps
  // before it takes the next ones, so a smaller grid means fewer tables in
  // flight: when all tables together exceed what the last-level cache holds well,
  // keep that many bytes in flight (but never less than three waves per compute unit).
  long resident = e->resident_envs;
  if (resident <= 0) {
    const size_t table_bytes = e->K * sizeof(float);
    resident = e->N;
    // (a launch of a few steps re-uses no row often enough for that to matter: it
    // runs with every env in flight)
    if ((size_t)e->N * table_bytes > kTableBytesInFlight && n_steps >= kInFlightMinSteps)
      resident = std::max<long>(kMinEnvsInFlight, (long)(kTableBytesInFlight / table_bytes));
    // The batch goes through the chip in shifts of that many envs; a last shift that
    // fills a fraction of the chip costs a whole one.  Even the shifts out, in whole
    // waves per compute unit (65,536 envs with 32x32 maps: 3.5e10 env-steps/s as one
    // shift of 49,152 and one of 16,384, 4.4e10 as two of 32,768).
    if (resident < e->N) {
      const long shifts = (e->N + resident - 1) / resident;
      const long per_shift = (e->N + shifts - 1) / shifts;
      const long unit = 64L * kComputeUnits;
      resident = std::min(resident, (per_shift + unit - 1) / unit * unit);
    }
  }
  p.tickets = p.map_kind == 0;
  const crl_config& c = e->cfg;
  // what the folded loop leaves out altogether ...
  const bool foldable = c.goal_mode == CRL_GOAL_ON_TARGET && c.auto_reset == 1 && c.max_mode == CRL_MAX_TRUE &&
                        e->trace_n == 0 && e->sup_n == 0 && c.max_episodes == 0 && c.track_returns == 0 &&
                        e->mv_words > 0;
  if (!p.tickets) {
    p.grid = (int)std::min<long>((e->N + p.block - 1) / p.block, std::max<long>(1, resident / p.block));
    // ... its variant for large or shared maps takes per-cell rewards and per-episode epsilon
    p.fast = foldable && c.eps_mode != CRL_EPS_STEP_MULT && c.table_mode != CRL_TABLE_SHARED;
    // two lanes per env while that still leaves the batch with at most two waves per
    // compute unit (config 5 with 8192 / 16,384 / 32,768 envs: +4 % / +6 % / -4 %)
    p.pair = p.fast && (e->N + 63) / 64 <= kComputeUnits;
    if (p.pair) p.grid = (int)std::min<long>((e->N + p.block / 2 - 1) / (p.block / 2), std::max<long>(1, 2 * resident / p.block));
  } else {
    p.rich = foldable && c.eps_mode != CRL_EPS_STEP_MULT && !(c.eps_mode == CRL_EPS_FIXED && c.reward_flags == 0);
    p.fast = foldable && c.eps_mode != CRL_EPS_STEP_MULT;
    // Hybrid workgroups when 32 whole tables (padded by one row against bank
    // conflicts), the LDS wave's maps and at least one table wave's maps fit into
    // LDS.  One workgroup per compute unit (the LDS holds no second one); the envs
    // in flight on HBM tables set how many 64-env waves work beside the LDS wave.
    p.tab_stride = (int)e->K + 4;
    const size_t map_lds = (size_t)e->map_words * 64 * 4;
    const size_t mv_lds = (size_t)e->mv_words * 64 * 4;
    const size_t lds_wave = p.fast ? (size_t)e->mv_words * crl::kTicketEnvs * 4 : map_lds;
    const size_t tables_lds = (size_t)crl::kTicketEnvs * p.tab_stride * 4;
    const long tickets = (e->N + crl::kTicketEnvs - 1) / crl::kTicketEnvs;
    // (not with per-cell rewards: they would stay in HBM, one request per step, and
    // a worker that waits for memory every step has no use for tables in LDS)
    const bool fits = e->K % 4 == 0 && map_lds + lds_wave + tables_lds <= kLdsPerWorkgroup && !p.rich;
    // ... and (automatic) when the tables outgrow the caches: while they all fit,
    // plain waves on every SIMD are faster (16x16 maps, env-steps/s plain / hybrid:
    // 32,768 envs 5.7e10 / 4.6e10, 65,536 envs 5.5e10 / 6.3e10, 262,144 envs 6.1e10 / 8.1e10)
    const bool outgrown = (size_t)e->N * e->K * sizeof(float) > kTableBytesInFlight;
    p.hybrid = fits && (e->fused_variant == 2 ||
                        (e->fused_variant == 0 && outgrown && n_steps >= kHybridMinSteps));
    if (p.hybrid) {
      p.grid = (int)std::min<long>(kComputeUnits, (tickets + 8) / 9);
      // at most three, so that the LDS wave has a SIMD to itself (1M envs, 8x8 / 12x12
      // maps: 1.11e11 / 1.00e11 env-steps/s with three table waves, 1.00e11 / 8.4e10 with four)
      long hbm_waves = std::min<long>(3, std::max<long>(1, resident / (64L * p.grid)));
      while (hbm_waves * map_lds + lds_wave + tables_lds > kLdsPerWorkgroup) --hbm_waves;
      p.block = 64 * ((int)hbm_waves + 1);
      p.lds = hbm_waves * map_lds + lds_wave + tables_lds;
    } else {
      long waves = 4, workers;  // waves per workgroup, 64-env workers in flight
      if (tickets / 2 < 4 * kComputeUnits) {
        // fewer 64-env workers than SIMDs on the chip: one-wave workgroups spread
        // them over the compute units instead of packing four per unit
        waves = 1;
        workers = std::min<long>(std::max<long>(1, resident / 64), (tickets + 1) / 2);
      } else if (resident <= 4L * 64 * kComputeUnits) {
        // at most four waves per compute unit: spread them over all units
        waves = std::max<long>(1, resident / (64L * kComputeUnits));
        workers = waves * std::min<long>(kComputeUnits, (tickets + 2 * waves - 1) / (2 * waves));
      } else {
        workers = 4 * std::min<long>(std::max<long>(1, resident / 256), (tickets + 7) / 8);
      }
      // every wave stages the maps of its 64 envs in its own LDS slice: large maps
      // leave room for fewer waves per workgroup (one always fits: map_kind 0
      // means 64 maps take at most 64 KB), the workers in flight stay the same
      while (waves > 1 && (size_t)waves * map_lds > kLdsPerWorkgroup) --waves;
      p.grid = (int)((workers + waves - 1) / waves);
      p.block = 64 * (int)waves;
      // staging the codes (four times the class map) pays off over a long launch only:
      // 1M envs of config 4, one step per launch 7.7e9 -> 1.4e10 with class maps, 48 steps 3.6e10 -> 3.7e10
      p.moves = p.fast && waves * mv_lds <= kLdsPerWorkgroup && n_steps >= kStagedMovesMinSteps;
      // Few enough envs that 32-env waves still find a SIMD each: one ticket per wave,
      // two lanes per env - half the distinct addresses per request and the Philox
      // rounds shared by the pair (32x32 maps: 4096 envs +10 %, 8192 +8 %, 16,384 +0 %)
      long units = tickets;  // tickets as the kernel counts them
      if (p.moves && waves == 1 && tickets <= 2 * kComputeUnits) {
        p.pair = true;
        // ... and thinner still while that gives more compute units a wave of their own
        // (4096 envs of 32x32: 128 waves of 32 envs 1.165e10 env-steps/s, 256 of 16 1.25e10,
        // 512 of 8 - two to a unit - 1.16e10)
        p.pair_envs = crl::kTicketEnvs;
        while (p.pair_envs > 8 && (e->N + p.pair_envs - 1) / p.pair_envs < kComputeUnits) p.pair_envs /= 2;
        units = (e->N + p.pair_envs - 1) / p.pair_envs;
        p.grid = (int)std::min<long>(std::max<long>(1, resident / p.pair_envs), units);
      }
      // Tickets dealt by position instead of drawn from a counter: the workers of this plan
      // all take the same time, and 16,384 draws from one counter take 0.38 ms however short
      // the launch (1M envs: the whole of a 4-step launch, half of a 20-step one).
      p.fixed = n_steps < kHybridMinSteps;
      (void)units;
      p.lds = waves * (p.moves ? mv_lds : map_lds);
    }
  }
  static const char* names[2][3][3] = {
      {{"k_fused_per_env<4,0>", "k_fused_per_env<4,1,general>", "k_fused_per_env<4,2,general>"},
       {"k_fused_per_env<4,0>", "k_fused_per_env<4,1,fast>", "k_fused_per_env<4,2,fast>"},
       {"k_fused_per_env<4,0>", "k_fused_per_env<4,1,fast,pairs>", "k_fused_per_env<4,2,fast,pairs>"}},
      {{"k_fused_per_env<8,0>", "k_fused_per_env<8,1,general>", "k_fused_per_env<8,2,general>"},
       {"k_fused_per_env<8,0>", "k_fused_per_env<8,1,fast>", "k_fused_per_env<8,2,fast>"},
       {"k_fused_per_env<8,0>", "k_fused_per_env<8,1,fast,pairs>", "k_fused_per_env<8,2,fast,pairs>"}}};
  p.name = names[e->A == 8][!p.fast ? 0 : p.pair ? 2 : 1][p.map_kind];
  if (p.tickets) {
    static const char* tnames[2][3][2] = {
        {{"k_fused_tickets<4,general,hbm>", "k_fused_tickets<4,general,hbm+lds>"},
         {"k_fused_tickets<4,fast,hbm>", "k_fused_tickets<4,fast,hbm+lds>"},
         {"k_fused_tickets<4,fast+,hbm>", "k_fused_tickets<4,fast+,hbm>"}},
        {{"k_fused_tickets<8,general,hbm>", "k_fused_tickets<8,general,hbm+lds>"},
         {"k_fused_tickets<8,fast,hbm>", "k_fused_tickets<8,fast,hbm+lds>"},
         {"k_fused_tickets<8,fast+,hbm>", "k_fused_tickets<8,fast+,hbm>"}}};
    p.name = tnames[e->A == 8][p.rich ? 2 : p.fast ? 1 : 0][p.hybrid];
  }
  return p;
}

template <int A>
void launch_fused_a(const crl_engine* e, const FusedPlan& p, uint64_t t0, int n) {
  const crl::Rules R = e->rules();
  const crl::Ptrs P = e->ptrs();
  if (p.tickets) {
    // (tickets dealt by position use no counter; the kernel itself notes who did how much)
    if (!p.fixed) hipLaunchKernelGGL(crl::k_fill_u32, dim3(1), dim3(64), 0, e->stream, e->tk, 0u, 3);
    const dim3 g(p.grid), b(p.block);
    unsigned* tk = e->tk;
#define CRL_LAUNCH_TICKETS(MODE, LDSW, MOVES)                                                       \
  hipLaunchKernelGGL((crl::k_fused_tickets<A, MODE, LDSW, MOVES>), g, b, p.lds, e->stream, R, P, t0, n, \
                     tk, p.tab_stride, p.fixed ? 1 : 0, p.pair ? p.pair_envs : 0)
    if (p.rich && p.moves)
      CRL_LAUNCH_TICKETS(2, false, true);
    else if (p.rich)
      CRL_LAUNCH_TICKETS(2, false, false);
    else if (p.fast && p.hybrid)
      CRL_LAUNCH_TICKETS(1, true, false);
    else if (p.fast && p.moves)
      CRL_LAUNCH_TICKETS(1, false, true);
    else if (p.fast)
      CRL_LAUNCH_TICKETS(1, false, false);
    else if (p.hybrid)
      CRL_LAUNCH_TICKETS(0, true, false);
    else
      CRL_LAUNCH_TICKETS(0, false, false);
#undef CRL_LAUNCH_TICKETS
    return;
  }
#define CRL_LAUNCH_PER_ENV(MAP, MODE)                                                                 \
  hipLaunchKernelGGL((crl::k_fused_per_env<A, MAP, MODE>), dim3(p.grid), dim3(p.block),               \
                     MAP == 1 ? p.lds : 0, e->stream, R, P, t0, n)
  const int mode = !p.fast ? 0 : p.pair ? 2 : 1;
  if (p.map_kind == 1) {
    if (mode == 2) CRL_LAUNCH_PER_ENV(1, 2);
    else if (mode == 1) CRL_LAUNCH_PER_ENV(1, 1);
    else CRL_LAUNCH_PER_ENV(1, 0);
  } else {
    if (mode == 2) CRL_LAUNCH_PER_ENV(2, 2);
    else if (mode == 1) CRL_LAUNCH_PER_ENV(2, 1);
    else CRL_LAUNCH_PER_ENV(2, 0);
  }
#undef CRL_LAUNCH_PER_ENV
}

constexpr size_t kHandoffLimitBytes = (size_t)128 << 20;

int ceil_log2(size_t v) {
  int b = 0;
  while (((size_t)1 << b) < v) ++b;
  return b;
}

crl::ReduceGeom reduce_geom(const crl_engine* e, int n) {
  crl::ReduceGeom G{};
  G.K = (int)e->K;
  G.a_shift = e->A == 8 ? 3 : 2;
  G.own_shift = ceil_log2((e->K + crl::kOwnKeys - 1) / crl::kOwnKeys);
  G.n_blocks = (n + crl::kBlockSamples - 1) / crl::kBlockSamples;
  G.cell_shift = crl::cell_shift_for(G.own_shift);
  G.main_shift = crl::main_shift_for(G.own_shift);
  return G;
}

size_t handoff_records(const crl::ReduceGeom& G) {
  return (((size_t)1 << G.own_shift) * (size_t)G.n_blocks) << G.cell_shift;
}

// the two-pass reduction needs the dense LDS table (K <= 16384) and a bounded hand-off buffer
bool reduce_fast(const crl_engine* e, const crl::ReduceGeom& G) {
  return e->K <= (size_t)crl::kDenseKeys && handoff_records(G) * sizeof(uint2) <= kHandoffLimitBytes;
}

constexpr size_t kOwnersLds = (size_t)(crl::kTileBlocks + crl::kTileBlocks / crl::kGroupBlocks) *
                              crl::kOwnKeys * sizeof(float) +
                              crl::kBlockSamples * sizeof(float);  // tile, group sums, a word per thread that nobody reads

template <class Kern>
hipError_t allow_lds(Kern kern, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// kernels that use more than the default 64 KB of LDS per workgroup (gfx950 has 160 KB)
int opt_in_lds(crl_engine* e) {
  if (e->lds_opt_in) return CRL_OK;
  const size_t act = kLdsPerWorkgroup;  // what a launch asks for is checked against this
  HIP_TRY(allow_lds(crl::k_reduce_blocks, crl::kReduceLdsBytes));
  HIP_TRY(allow_lds(crl::k_reduce_owners, kOwnersLds));
  HIP_TRY(allow_lds(crl::k_shared_act<4, 1, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_act<4, 2, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_act<8, 1, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_act<8, 2, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 1, false, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 1, false, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 2, false, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 2, false, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 1, false, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 1, false, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 2, false, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 2, false, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 1, true, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 1, true, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 2, true, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<4, 2, true, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 1, true, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 1, true, true>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 2, true, false>, act - kStaticLdsReserve));
  HIP_TRY(allow_lds(crl::k_shared_persist<8, 2, true, true>, act - kStaticLdsReserve));
  e->lds_opt_in = true;
  return CRL_OK;
}

// the hand-off cells fit where this call may keep them
bool handoff_fits(const crl_engine* e, const crl::ReduceGeom& G) {
  return !e->no_alloc || handoff_records(G) * sizeof(unsigned long long) <= kScratchExchangeBytes;
}

int ensure_handoff(crl_engine* e, const crl::ReduceGeom& G) {
  const size_t recs = handoff_records(G);
  if (e->no_alloc) {
    if (!handoff_fits(e, G))
      return fail(CRL_E_RANGE, "the ordered reduction of this engine needs %zu bytes of hand-off cells, "
                  "the static scratch of crl_run_fused_noalloc holds %zu", recs * sizeof(unsigned long long),
                  kScratchExchangeBytes);
    e->ho = reinterpret_cast<unsigned long long*>(e->static_scratch + kScratchTicketBytes);
  } else {
    hipError_t h = e->handoff.ensure(recs);
    if (h != hipSuccess) return fail(CRL_E_ALLOC, "hand-off buffer allocation failed: %s", hipGetErrorString(h));
    e->ho = e->handoff.p;
  }
  return opt_in_lds(e);
}

int reduce_owners(crl_engine* e, const crl::ReduceGeom& G, float* Q, const int32_t* key,
                  const float* delta, int n) {
  hipLaunchKernelGGL(crl::k_reduce_owners, dim3(1 << G.own_shift), dim3(256), kOwnersLds, e->stream, G,
                     Q, key, delta, n, e->ho);
  HIP_TRY(hipGetLastError());
  return CRL_OK;
}

// Q[k] += ordered sum of delta[i] with key[i] == k, for n samples on one table
int reduce_apply(crl_engine* e, float* Q, const int32_t* key, const float* delta, int n) {
  const crl::ReduceGeom G = reduce_geom(e, n);
  e->no_alloc = false;  // crl_update / crl_td_update: the engine's own hand-off buffer
  if (!reduce_fast(e, G)) {
    const int grid = (int)((e->K + crl::kOwnKeys - 1) / crl::kOwnKeys);
    hipLaunchKernelGGL(crl::k_reduce_scan, dim3(grid), dim3(256), 0, e->stream, Q, (int)e->K, key,
                       delta, n);
    HIP_TRY(hipGetLastError());
    return CRL_OK;
  }
  int rc = ensure_handoff(e, G);
  if (rc) return rc;
  hipLaunchKernelGGL(crl::k_reduce_blocks, dim3(G.n_blocks), dim3(crl::kBlockSamples),
                     crl::kReduceLdsBytes, e->stream, G, key, delta, n, e->ho);
  HIP_TRY(hipGetLastError());
  return reduce_owners(e, G, Q, key, delta, n);
}

template <int A, int MAP>
void launch_shared_act(crl_engine* e, bool reduce, const crl::ReduceGeom& G, uint64_t t, int trace_row) {
  const crl::Rules R = e->rules();
  const crl::Ptrs P = e->ptrs();
  const int block = 256, grid = (e->N + block - 1) / block;
  const size_t lds = (reduce ? crl::kReduceLdsBytes : 0) + (MAP == 1 ? (size_t)e->map_words * 4 : 0);
  if (reduce)
    hipLaunchKernelGGL((crl::k_shared_act<A, MAP, true>), dim3(grid), dim3(block), lds, e->stream, R, P,
                       t, trace_row, e->key.p, e->delta.p, G, e->ho);
  else
    hipLaunchKernelGGL((crl::k_shared_act<A, MAP, false>), dim3(grid), dim3(block), lds, e->stream, R,
                       P, t, trace_row, e->key.p, e->delta.p, G, e->ho);
}

// one shared-table step: act (select + move + delta + block sums), then the key owners
int shared_step(crl_engine* e, uint64_t t, int trace_row) {
  const crl::ReduceGeom G = reduce_geom(e, e->N);
  const bool fast = reduce_fast(e, G);
  if (fast) {
    int rc = ensure_handoff(e, G);
    if (rc) return rc;
  }
  // LDS plan of the act kernel: reduction table (fast path), then the map.  The
  // shared table itself stays in L2: streaming its 64 KB into every workgroup's
  // LDS each step measured slower than the row reads it saves (12.4 against 12.05 us
  // per step on 65,536 envs, also against the five speculative reads per env).
  size_t lds = fast ? crl::kReduceLdsBytes : 0;
  const size_t limit = fast ? kLdsPerWorkgroup - kStaticLdsReserve : (size_t)64 * 1024;
  const size_t map_bytes = (size_t)e->map_words * 4;
  const bool lds_map = e->cfg.map_mode == CRL_MAP_SHARED && map_bytes <= (size_t)kLdsMapLimitBytes &&
                       lds + map_bytes <= limit;
  if (lds_map) lds += map_bytes;
  if (e->A == 4) {
    if (lds_map) launch_shared_act<4, 1>(e, fast, G, t, trace_row);
    else launch_shared_act<4, 2>(e, fast, G, t, trace_row);
  } else {
    if (lds_map) launch_shared_act<8, 1>(e, fast, G, t, trace_row);
    else launch_shared_act<8, 2>(e, fast, G, t, trace_row);
  }
  HIP_TRY(hipGetLastError());
  if (fast) return reduce_owners(e, G, e->Q.p, e->key.p, e->delta.p, e->N);
  const int grid = (int)((e->K + crl::kOwnKeys - 1) / crl::kOwnKeys);
  hipLaunchKernelGGL(crl::k_reduce_scan, dim3(grid), dim3(256), 0, e->stream, e->Q.p, (int)e->K,
                     e->key.p, e->delta.p, e->N);
  HIP_TRY(hipGetLastError());
  return CRL_OK;
}

// ---- shared table: all steps of a call in one launch ---------------------------------

struct PersistPlan {
  bool ok;
  int grid;
  bool lds_map;
  bool fold;  // the instantiation with the common configuration's rules folded in
  size_t lds;
  crl::ReduceGeom G;
  // what the workgroups exchange, in 64-bit words from the start of one buffer
  size_t at_table, at_raw, at_cells, words;
};

// Shortest call worth the set-up of the one-launch kernel (clearing what its workgroups
// exchange, one co-resident launch) instead of two plain launches per step.
constexpr int kPersistMinSteps = 4;

// The one-launch kernel needs every workgroup resident at once (one per compute
// unit), the dense LDS table of the block pass and one tile of the owners' pass.
PersistPlan plan_persist(const crl_engine* e, int n_steps) {
  PersistPlan p{};
  if (e->cfg.table_mode != CRL_TABLE_SHARED || e->fused_variant == 1 || e->persist_refused) return p;
  if (e->fused_variant == 0 && n_steps < kPersistMinSteps) return p;
  const int n_blocks = (e->N + crl::kBlockSamples - 1) / crl::kBlockSamples;
  if (e->K > (size_t)crl::kDenseKeys || n_blocks > crl::kPersistMaxGroups || crl::kPersistMaxGroups > kComputeUnits) return p;
  // always 256 workgroups, each a block (with or without envs) and an owner (with or
  // without keys): 16,384 keys at most are 64 to an owner
  p.G = reduce_geom(e, e->N);
  p.G.own_shift = crl::kPersistOwnShift;
  p.G.cell_shift = crl::cell_shift_for(p.G.own_shift);
  p.G.main_shift = crl::main_shift_for(p.G.own_shift);
  p.grid = crl::kPersistMaxGroups;
  p.G.n_blocks = p.grid;  // workgroups without envs hand over empty cells
  const crl_config& c = e->cfg;
  p.fold = c.goal_mode == CRL_GOAL_ON_TARGET && c.auto_reset == 1 && c.max_mode == CRL_MAX_TRUE && c.reward_flags == 0 &&
           e->trace_n == 0 && e->sup_n == 0 && c.max_episodes == 0 && c.track_returns == 0;
  const int n_own = 1 << p.G.own_shift;
  const size_t map_bytes = (size_t)e->map_words * 4;
  p.lds_map = e->cfg.map_mode == CRL_MAP_SHARED && sizeof(crl::PersistLds) + map_bytes <= kLdsPerWorkgroup - kStaticLdsReserve;
  p.lds = sizeof(crl::PersistLds) + (p.lds_map ? map_bytes : 0);
  auto pad = [](size_t words) { return (words + 31) & ~(size_t)31; };  // 256-byte pieces
  p.at_table = 0;
  p.at_raw = p.at_table + pad(2 * (size_t)e->K);  // a cell's view: its A values and A neighbours' maxima
  p.at_cells = p.at_raw + pad(2 * (size_t)e->N);  // raw samples and cells: two buffers each
  p.words = p.at_cells + 2 * (((size_t)n_own * p.grid) << p.G.cell_shift);
  if (e->no_alloc && p.words * sizeof(unsigned long long) > kScratchExchangeBytes) return p;
  p.ok = true;
  return p;
}

template <int A, int MAP, bool CLK, bool FOLD>
hipError_t launch_persist_kernel(crl_engine* e, const PersistPlan& p, unsigned long long* buf, uint64_t t0,
                                 int n_steps, int trace_row0) {
  crl::Rules R = e->rules();
  crl::Ptrs P = e->ptrs();
  crl::ReduceGeom G = p.G;
  crl::PersistBufs B{};
  B.table = buf + p.at_table;
  B.raw = buf + p.at_raw;
  B.cells = buf + p.at_cells;
  B.err = reinterpret_cast<unsigned*>(e->pdiag.p);
  B.clocks = e->pdiag.p + 1;
  int spin_limit = e->persist_spin_limit;
  void* args[] = {&R, &P, &t0, &n_steps, &trace_row0, &G, &B, &spin_limit};
  // a cooperative launch is refused unless all workgroups can be resident together,
  // which the kernel's waits rely on
  return hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&crl::k_shared_persist<A, MAP, CLK, FOLD>), dim3(p.grid),
                                    dim3(256), args, (unsigned)p.lds, e->stream);
}

static_assert(crl::kPersistClockWords == CRL_PERSIST_CLOCK_WORDS, "include/crl.h states the size of the diagnostics");

// -> CRL_OK and *launched = true, or *launched = false when the caller should take
// the two-launches-per-step path instead
int run_persist(crl_engine* e, int n_steps, bool* launched) {
  *launched = false;
  const PersistPlan p = plan_persist(e, n_steps);
  if (!p.ok) return CRL_OK;
  int rc;
  unsigned long long* buf;
  if (e->no_alloc) {
    buf = reinterpret_cast<unsigned long long*>(e->static_scratch + kScratchTicketBytes);
  } else {
    if (e->pbuf.ensure(p.words) != hipSuccess) return fail(CRL_E_ALLOC, "allocation of the exchange buffers failed");
    buf = e->pbuf.p;
  }
  rc = opt_in_lds(e);
  if (rc) return rc;
  // The kernel's tags count the steps of one launch, so everything the workgroups
  // exchange starts from tag 0 (a fill kernel, not a memset: a caller may record this),
  // and a call longer than the tags allow goes out as several launches.
  int done = 0;
  while (done < n_steps) {
    const int n = std::min(n_steps - done, crl::kPersistMaxSteps);
    const size_t w32 = p.words * 2;
    hipLaunchKernelGGL(crl::k_fill_u32, dim3((unsigned)((w32 + 255) / 256)), dim3(256), 0, e->stream,
                       reinterpret_cast<unsigned*>(buf), 0u, w32);
    const uint64_t t0 = e->t + (uint64_t)done;
    const int row0 = (int)std::min<long long>((long long)e->trace_cursor + done, e->trace_cap);
    hipError_t h;
#define CRL_PERSIST(A, MAP) \
  (e->persist_clocks ? (p.fold ? launch_persist_kernel<A, MAP, true, true>(e, p, buf, t0, n, row0)    \
                               : launch_persist_kernel<A, MAP, true, false>(e, p, buf, t0, n, row0))  \
                     : (p.fold ? launch_persist_kernel<A, MAP, false, true>(e, p, buf, t0, n, row0)   \
                               : launch_persist_kernel<A, MAP, false, false>(e, p, buf, t0, n, row0)))
    if (e->A == 4) h = p.lds_map ? CRL_PERSIST(4, 1) : CRL_PERSIST(4, 2);
    else h = p.lds_map ? CRL_PERSIST(8, 1) : CRL_PERSIST(8, 2);
#undef CRL_PERSIST
    if (h != hipSuccess) {
      (void)hipGetLastError();
      if (done > 0) return fail(CRL_E_DEVICE, "the one-launch shared-table kernel was refused after %d steps: %s", done, hipGetErrorString(h));
      e->persist_refused = true;  // not resident all at once on this device: never mind, two launches per step
      return CRL_OK;
    }
    e->persist_unchecked = true;
    done += n;
  }
  if (e->trace_n > 0) {
    const long long c = (long long)e->trace_cursor + n_steps;
    e->trace_cursor = c > e->trace_cap ? e->trace_cap : (int)c;
  }
  *launched = true;
  return CRL_OK;
}

// Did a one-launch kernel give up waiting for its peers?  Called by the entry points
// that synchronise; reports a give-up once.  The give-up word stays set on the device
// (the kernel's later launches see it and return at once), and until the caller has set
// state or table again every call that works on them fails (require_valid).
int check_persist(crl_engine* e) {
  if (!e->persist_unchecked) return CRL_OK;
  e->persist_unchecked = false;
  unsigned gave_up = 0;
  HIP_TRY(hipMemcpyAsync(&gave_up, e->pdiag.p, sizeof gave_up, hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  if (!gave_up) return CRL_OK;
  e->persist_failed = true;
  return fail(CRL_E_DEVICE, "the one-launch shared-table kernel gave up waiting for its workgroups "
              "(were they all resident?); state and table are not valid: set them again (crl_reset, "
              "crl_set_state, crl_q_set) and use crl_set_fused_variant(e, 1)");
}

int require_valid(const crl_engine* e) {
  if (e->persist_failed)
    return fail(CRL_E_STATE, "a one-launch shared-table kernel gave up earlier: state and table are not valid "
                "until crl_reset, crl_set_state or crl_q_set");
  return CRL_OK;
}

// The caller sets state or table again.  A launch nobody has looked at yet is looked at
// first (and a give-up reported by this call); a give-up already reported is history.
int clear_persist_failure(crl_engine* e) {
  int rc = check_persist(e);
  if (rc) return rc;
  if (!e->persist_failed) return CRL_OK;
  HIP_TRY(hipMemsetAsync(e->pdiag.p, 0, sizeof(unsigned long long), e->stream));
  e->persist_failed = false;
  return CRL_OK;
}

// sizes that follow from the configuration alone
void set_geometry(crl_engine* e, const crl_config& cfg) {
  e->cfg = cfg;
  e->N = cfg.n_envs;
  e->W = cfg.width;
  e->H = cfg.height;
  e->A = cfg.n_actions;
  e->S = (size_t)cfg.width * cfg.height;
  e->K = e->S * e->A;
  e->n_maps = cfg.map_mode == CRL_MAP_SHARED ? 1 : e->N;
  e->n_tables = cfg.table_mode == CRL_TABLE_SHARED ? 1 : e->N;
  e->map_words = (int)((e->S + 15) / 16);
  const size_t cells_per_word = 16 / (size_t)e->A;
  e->mv_words = (int)((e->S + cells_per_word - 1) / cells_per_word);
}

int check_engine(const crl_engine* e) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  hipError_t err = hipSetDevice(e->device);
  if (err != hipSuccess) return fail(CRL_E_DEVICE, "hipSetDevice(%d): %s", e->device, hipGetErrorString(err));
  return CRL_OK;
}

int check_usable(const crl_engine* e) {
  int rc = check_engine(e);
  return rc ? rc : require_valid(e);
}

// move codes of maps [first, first + count) from the class maps on the device
int build_moves(crl_engine* e, int first, int count) {
  if (e->mv_words == 0 || count <= 0) return CRL_OK;
  const size_t threads = (size_t)count * e->mv_words;
  const dim3 g((unsigned)((threads + 255) / 256)), b(256);
  if (e->A == 4)
    hipLaunchKernelGGL(crl::k_build_moves<4>, g, b, 0, e->stream, e->map.p, e->map_words, e->W, e->H,
                       e->mv_words, first, count, e->moves.p);
  else
    hipLaunchKernelGGL(crl::k_build_moves<8>, g, b, 0, e->stream, e->map.p, e->map_words, e->W, e->H,
                       e->mv_words, first, count, e->moves.p);
  HIP_TRY(hipGetLastError());
  return CRL_OK;
}

// Packs the caller's class maps 2 bits to a cell and uploads them a slice of maps at a
// time (the engine keeps no host copy of maps or cell rewards: for 8192 maps of 256x256
// cells those would be 0.5 GB and 2 GB for the life of the engine).
int upload_maps(crl_engine* e, const uint8_t* cell_class, const float* cell_reward) {
  const size_t slice_maps = std::max<size_t>(1, ((size_t)16 << 20) / ((size_t)e->map_words * 4));
  std::vector<uint32_t> packed(std::min<size_t>(slice_maps, (size_t)e->n_maps) * e->map_words);
  for (size_t m0 = 0; m0 < (size_t)e->n_maps; m0 += slice_maps) {
    const size_t count = std::min(slice_maps, (size_t)e->n_maps - m0);
    std::fill(packed.begin(), packed.end(), 0u);
    for (size_t m = 0; m < count; ++m)
      crl::pack_classes(cell_class + (m0 + m) * e->S, e->S, packed.data() + m * e->map_words);
    HIP_TRY(hipMemcpyAsync(e->map.p + m0 * e->map_words, packed.data(), count * e->map_words * sizeof(uint32_t),
                           hipMemcpyHostToDevice, e->stream));
    HIP_TRY(hipStreamSynchronize(e->stream));  // the slice buffer is filled again next round
  }
  if (e->cfg.reward_flags & CRL_REWARD_CELLS)
    HIP_TRY(hipMemcpyAsync(e->cell_reward.p, cell_reward, (size_t)e->n_maps * e->S * sizeof(float),
                           hipMemcpyHostToDevice, e->stream));
  const int rc = build_moves(e, 0, e->n_maps);
  if (rc) return rc;
  HIP_TRY(hipStreamSynchronize(e->stream));
  return CRL_OK;
}

int opt_in_ticket_kernels(crl_engine* e);

int create_engine(const crl_config* cfg, int device, crl_engine** out) {
  if (!out) return fail(CRL_E_ARG, "out is null");
  *out = nullptr;
  int rc = crl::validate_config(cfg, crl::last_error());
  if (rc != CRL_OK) return rc;
  int ndev = 0;
  hipError_t herr = hipGetDeviceCount(&ndev);
  if (herr != hipSuccess || ndev <= 0)
    return fail(CRL_E_DEVICE, "no HIP device available (%s); this engine has no CPU path",
                herr != hipSuccess ? hipGetErrorString(herr) : "count is 0");
  if (device < 0 || device >= ndev) return fail(CRL_E_ARG, "device %d out of range [0,%d)", device, ndev);
  HIP_TRY(hipSetDevice(device));

  std::unique_ptr<crl_engine> own(new crl_engine());  // freed on every early return and on a throw
  crl_engine* e = own.get();
  set_geometry(e, *cfg);
  e->device = device;

  const size_t N = (size_t)e->N;
  std::vector<float> eps = crl::build_eps_table(*cfg);
  e->eps_len = (int)eps.size();
  const bool cells = (cfg->reward_flags & CRL_REWARD_CELLS) != 0;
  hipError_t a = hipSuccess;
  auto acc = [&](hipError_t x) {
    if (a == hipSuccess) a = x;
  };
  acc(e->s.alloc(N));
  acc(e->ep_step.alloc(N));
  acc(e->episode.alloc(N));
  acc(e->start.alloc(N));
  acc(e->act.alloc(N));
  acc(e->reward.alloc(N));
  acc(e->done.alloc(N));
  acc(e->action.alloc(N));
  acc(e->map.alloc((size_t)e->n_maps * e->map_words));
  acc(e->moves.alloc((size_t)e->n_maps * e->mv_words));  // move codes of every map, for the fused loops
  if (cells) acc(e->cell_reward.alloc((size_t)e->n_maps * e->S));
  acc(e->Q.alloc((size_t)e->n_tables * e->K));
  acc(e->eps_tab.alloc(eps.size()));
  acc(e->tr_s.alloc(N));
  acc(e->tr_a.alloc(N));
  acc(e->tr_s2.alloc(N));
  acc(e->tr_r.alloc(N));
  acc(e->tr_done.alloc(N));
  if (cfg->table_mode == CRL_TABLE_PER_ENV) acc(e->split.alloc(3));
  if (cfg->table_mode == CRL_TABLE_SHARED) {
    acc(e->key.alloc(N));
    acc(e->delta.alloc(N));
    acc(e->pdiag.alloc(1 + crl::kPersistClockWords));
  }
  if (cfg->track_returns) {
    acc(e->ret_acc.alloc(N));
    acc(e->ret_last.alloc(N));
    acc(e->ret_sum.alloc(N));
    acc(e->len_last.alloc(N));
    acc(e->len_sum.alloc(N));
  }
  if (a != hipSuccess) {
    const int code = a == hipErrorOutOfMemory ? CRL_E_ALLOC : CRL_E_DEVICE;
    return fail(code, "device allocation failed: %s", hipGetErrorString(a));
  }
  auto bail = [&](hipError_t x, const char* what) {
    return fail(CRL_E_DEVICE, "%s: %s", what, hipGetErrorString(x));
  };
  hipError_t h;
  if ((h = hipMemsetAsync(e->Q.p, 0, e->Q.n * sizeof(float), e->stream)) != hipSuccess)
    return bail(h, "clear Q");
  if ((h = hipMemsetAsync(e->s.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear s");
  if ((h = hipMemsetAsync(e->ep_step.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->episode.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->start.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->act.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->reward.p, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->done.p, 0, N, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->action.p, 0, N, e->stream)) != hipSuccess) return bail(h, "clear");
  if ((h = hipMemsetAsync(e->map.p, 0, e->map.n * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  if (e->pdiag.p && (h = hipMemsetAsync(e->pdiag.p, 0, e->pdiag.n * 8, e->stream)) != hipSuccess) return bail(h, "clear");
  if (cfg->track_returns) {
    void* bufs[] = {e->ret_acc.p, e->ret_last.p, e->ret_sum.p, e->len_last.p, e->len_sum.p};
    for (void* b : bufs)
      if ((h = hipMemsetAsync(b, 0, N * 4, e->stream)) != hipSuccess) return bail(h, "clear");
  }
  if ((h = hipMemcpyAsync(e->eps_tab.p, eps.data(), eps.size() * sizeof(float), hipMemcpyHostToDevice,
                          e->stream)) != hipSuccess)
    return bail(h, "upload eps table");
  if (cells) {  // until crl_set_maps: every cell pays the step reward
    uint32_t bits;
    std::memcpy(&bits, &cfg->step_reward, 4);
    const size_t n = e->cell_reward.n;
    hipLaunchKernelGGL(crl::k_fill_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, e->stream,
                       reinterpret_cast<unsigned*>(e->cell_reward.p), bits, n);
    if ((h = hipGetLastError()) != hipSuccess) return bail(h, "fill cell rewards");
  }
  if ((h = hipStreamSynchronize(e->stream)) != hipSuccess) return bail(h, "sync");
  // set-up that crl_run_fused_noalloc must not have left to do: this device's copy
  // of the scratch array, and the kernels that may use the whole LDS
  rc = scratch_of_device(device, &e->static_scratch);
  if (rc == CRL_OK) rc = cfg->table_mode == CRL_TABLE_SHARED ? opt_in_lds(e) : opt_in_ticket_kernels(e);
  if (rc != CRL_OK) return rc;
  *out = own.release();
  return CRL_OK;
}

int reset_envs(crl_engine* e, int32_t first, int32_t count) {
  int rc = check_engine(e);
  if (rc) return rc;
  rc = clear_persist_failure(e);
  if (rc) return rc;
  if (first < 0 || count < 0 || (int64_t)first + count > e->N)
    return fail(CRL_E_RANGE, "env range [%d,%d) outside [0,%d)", first, first + count, e->N);
  if (count == 0) return CRL_OK;
  hipLaunchKernelGGL(crl::k_reset, dim3((count + 255) / 256), dim3(256), 0, e->stream, e->ptrs(), first,
                     count);
  HIP_TRY(hipGetLastError());
  e->have_transition = false;
  return CRL_OK;
}

int set_maps(crl_engine* e, const uint8_t* cell_class, const int32_t* start,
                 const float* cell_reward) {
  int rc = check_engine(e);
  if (rc) return rc;
  if (!cell_class) return fail(CRL_E_ARG, "cell_class is null");
  const bool cells = (e->cfg.reward_flags & CRL_REWARD_CELLS) != 0;
  if (cells && !cell_reward) return fail(CRL_E_ARG, "reward_flags asks for cell rewards but none given");
  if (!cells && cell_reward) return fail(CRL_E_ARG, "cell rewards given but reward_flags has no CRL_REWARD_CELLS");
  const size_t total = (size_t)e->n_maps * e->S;
  for (size_t i = 0; i < total; ++i)
    if (cell_class[i] > CRL_CELL_WALL) return fail(CRL_E_ARG, "cell_class[%zu] = %d is not a cell class", i, (int)cell_class[i]);
  if (start)
    for (int i = 0; i < e->N; ++i)
      if (start[i] < 0 || (size_t)start[i] >= e->S)
        return fail(CRL_E_RANGE, "start[%d] = %d outside [0,%zu)", i, start[i], e->S);
  rc = upload_maps(e, cell_class, cell_reward);
  if (rc) return rc;
  if (start) {
    HIP_TRY(hipMemcpyAsync(e->start.p, start, (size_t)e->N * 4, hipMemcpyHostToDevice, e->stream));
    HIP_TRY(hipStreamSynchronize(e->stream));
  }
  return reset_envs(e, 0, e->N);
}

int set_cell(crl_engine* e, int32_t map_index, int32_t cell, int32_t cell_class,
                 float cell_reward) {
  int rc = check_engine(e);
  if (rc) return rc;
  if (map_index < 0 || map_index >= e->n_maps) return fail(CRL_E_RANGE, "map index %d outside [0,%d)", map_index, e->n_maps);
  if (cell < 0 || (size_t)cell >= e->S) return fail(CRL_E_RANGE, "cell %d outside [0,%zu)", cell, e->S);
  if (cell_class < CRL_CELL_FREE || cell_class > CRL_CELL_WALL) return fail(CRL_E_ARG, "%d is not a cell class", cell_class);
  const size_t at = (size_t)map_index * e->S + cell;
  // the word of 16 cells that holds this one: fetched, changed, put back
  const size_t word = (size_t)map_index * e->map_words + (cell >> 4);
  uint32_t packed = 0;
  HIP_TRY(hipMemcpyAsync(&packed, e->map.p + word, 4, hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  const int shift = 2 * (cell & 15);
  packed = (packed & ~(3u << shift)) | ((uint32_t)cell_class << shift);
  HIP_TRY(hipMemcpyAsync(e->map.p + word, &packed, 4, hipMemcpyHostToDevice, e->stream));
  rc = build_moves(e, map_index, 1);  // the neighbours' codes name this cell
  if (rc) return rc;
  if (e->cfg.reward_flags & CRL_REWARD_CELLS)
    HIP_TRY(hipMemcpyAsync(e->cell_reward.p + at, &cell_reward, 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));  // `packed` and `cell_reward` are this call's
  return CRL_OK;
}

// every ticket-kernel instantiation launch_fused_a can pick may use the whole LDS:
// the plain ones, too, ask for more than the default 64 KB when large per-env
// maps share a workgroup
int opt_in_ticket_kernels(crl_engine* e) {
  if (e->hybrid_opt_in) return CRL_OK;
  const void* fns[] = {
#define CRL_TICKET_KERNELS(A)                                                          \
  reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 0, false, false>),            \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 1, false, false>),        \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 2, false, false>),        \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 0, true, false>),         \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 1, true, false>),         \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 1, false, true>),         \
      reinterpret_cast<const void*>(&crl::k_fused_tickets<A, 2, false, true>)
      CRL_TICKET_KERNELS(4), CRL_TICKET_KERNELS(8)
#undef CRL_TICKET_KERNELS
  };
  for (const void* fn : fns)
    HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerWorkgroup));
  e->hybrid_opt_in = true;
  return CRL_OK;
}

// crl_run_fused and its allocation-free variant: with `no_alloc` the ticket
// counters and the hand-off cells live in the device's static scratch array and
// nothing below allocates or frees
int run_fused(crl_engine* e, int32_t n_steps, bool no_alloc) {
  int rc = check_engine(e);
  if (rc) return rc;
  if (n_steps < 0) return fail(CRL_E_ARG, "negative step count");
  if (n_steps == 0) return CRL_OK;
  if (no_alloc && !e->static_scratch) return fail(CRL_E_STATE, "the device's scratch array was not found at crl_create");
  rc = require_valid(e);
  if (rc) return rc;
  // whichever way this call ends, later calls work with the engine's own buffers again
  struct Restore {
    crl_engine* e;
    ~Restore() { e->no_alloc = false; }
  } restore{e};
  e->no_alloc = no_alloc;
  if (e->cfg.table_mode == CRL_TABLE_PER_ENV) {
    const FusedPlan p = plan_fused(e, n_steps);
    if (p.lds > kLdsPerWorkgroup)
      return fail(CRL_E_STATE, "launch plan %s needs %zu bytes of LDS per workgroup, the device has %zu",
                  p.name, p.lds, kLdsPerWorkgroup);
    if (p.tickets) {
      if (no_alloc) {
        e->tk = reinterpret_cast<unsigned*>(e->static_scratch);
      } else {
        if (e->ticket.ensure(3) != hipSuccess) return fail(CRL_E_ALLOC, "ticket counter allocation failed");
        e->tk = e->ticket.p;
      }
      rc = opt_in_ticket_kernels(e);  // done at crl_create; a no-op here
      if (rc) return rc;
    }
    if (e->A == 4)
      launch_fused_a<4>(e, p, e->t, n_steps);
    else
      launch_fused_a<8>(e, p, e->t, n_steps);
    HIP_TRY(hipGetLastError());
    if (p.tickets) {
      // the counters may sit in the scratch all engines of this GPU share: kept here
      hipLaunchKernelGGL(crl::k_copy3_u32, dim3(1), dim3(64), 0, e->stream, e->tk, e->split.p);
      HIP_TRY(hipGetLastError());
    }
    e->split_valid = p.tickets;
    if (e->trace_n > 0) {
      const long long c = (long long)e->trace_cursor + n_steps;
      e->trace_cursor = c > e->trace_cap ? e->trace_cap : (int)c;
    }
  } else {
    bool launched = false;
    rc = run_persist(e, n_steps, &launched);
    if (rc) return rc;
    for (int k = 0; !launched && k < n_steps; ++k) {
      rc = shared_step(e, e->t + (uint64_t)k, e->trace_cursor);
      if (rc) return rc;
      if (e->trace_n > 0 && e->trace_cursor < e->trace_cap) e->trace_cursor += 1;
    }
  }
  e->t += (uint64_t)n_steps;
  e->have_transition = false;
  e->have_actions = false;
  return CRL_OK;
}

}  // namespace

extern "C" {

const char* crl_last_error(void) { return crl::last_error().c_str(); }
const char* crl_version(void) { return CRL_VERSION; }

int crl_device_count(void) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) return fail(CRL_E_DEVICE, "hipGetDeviceCount: %s", hipGetErrorString(e));
  return n;
}

int crl_create(const crl_config* cfg, int device, crl_engine** out) {
  return guarded([&] { return create_engine(cfg, device, out); });
}

int crl_destroy(crl_engine* e) {
  if (!e) return CRL_OK;
  (void)hipSetDevice(e->device);
  (void)hipStreamSynchronize(e->stream);
  delete e;
  return CRL_OK;
}

int crl_set_stream(crl_engine* e, void* hip_stream) {
  int rc = check_engine(e);
  if (rc) return rc;
  HIP_TRY(hipStreamSynchronize(e->stream));
  e->stream = reinterpret_cast<hipStream_t>(hip_stream);
  return CRL_OK;
}

int crl_set_resident_envs(crl_engine* e, int32_t n_envs) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  if (n_envs < 0) return fail(CRL_E_ARG, "negative env count");
  e->resident_envs = n_envs;
  return CRL_OK;
}

int crl_set_fused_variant(crl_engine* e, int32_t variant) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  if (variant < 0 || variant > 2) return fail(CRL_E_ARG, "variant must be 0 (automatic), 1 or 2");
  e->fused_variant = variant;
  return CRL_OK;
}

int crl_get_fused_split(crl_engine* e, uint32_t* hbm_envs, uint32_t* lds_envs) {
  int rc = check_usable(e);
  if (rc) return rc;
  unsigned v[3] = {0, 0, 0};
  if (e->split_valid) {
    HIP_TRY(hipMemcpyAsync(v, e->split.p, sizeof v, hipMemcpyDeviceToHost, e->stream));
    HIP_TRY(hipStreamSynchronize(e->stream));
  }
  if (hbm_envs) *hbm_envs = v[1];
  if (lds_envs) *lds_envs = v[2];
  return CRL_OK;
}

int crl_sync(crl_engine* e) {
  int rc = check_engine(e);
  if (rc) return rc;
  HIP_TRY(hipStreamSynchronize(e->stream));
  return check_persist(e);
}

int crl_set_maps(crl_engine* e, const uint8_t* cell_class, const int32_t* start,
                 const float* cell_reward) {
  return guarded([&] { return set_maps(e, cell_class, start, cell_reward); });
}

int crl_set_cell(crl_engine* e, int32_t map_index, int32_t cell, int32_t cell_class,
                 float cell_reward) {
  return guarded([&] { return set_cell(e, map_index, cell, cell_class, cell_reward); });
}

int crl_reset(crl_engine* e, int32_t first, int32_t count) { return reset_envs(e, first, count); }

int crl_step(crl_engine* e, const int32_t* actions) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (actions) {
    HIP_TRY(hipMemcpyAsync(e->act.p, actions, (size_t)e->N * 4, hipMemcpyHostToDevice, e->stream));
    // the host buffer may be reused as soon as we return
    HIP_TRY(hipStreamSynchronize(e->stream));
  } else if (!e->have_actions) {
    return fail(CRL_E_STATE, "crl_step(NULL) needs a preceding crl_select");
  }
  hipLaunchKernelGGL(crl::k_step, dim3((e->N + 255) / 256), dim3(256), 0, e->stream, e->rules(),
                     e->ptrs(), e->transition(), e->act.p);
  HIP_TRY(hipGetLastError());
  if (e->trace_n > 0 && e->trace_cursor < e->trace_cap) e->trace_cursor += 1;
  e->have_transition = true;
  e->have_actions = false;
  return CRL_OK;
}

int crl_select(crl_engine* e, int32_t* actions_out) {
  int rc = check_usable(e);
  if (rc) return rc;
  const long long threads = (long long)e->N * e->A;
  const int grid = (int)((threads + 255) / 256);
  if (e->A == 4)
    hipLaunchKernelGGL((crl::k_select<4>), dim3(grid), dim3(256), 0, e->stream, e->rules(), e->ptrs(),
                       e->t, e->act.p);
  else
    hipLaunchKernelGGL((crl::k_select<8>), dim3(grid), dim3(256), 0, e->stream, e->rules(), e->ptrs(),
                       e->t, e->act.p);
  HIP_TRY(hipGetLastError());
  e->have_actions = true;
  if (actions_out) {
    HIP_TRY(hipMemcpyAsync(actions_out, e->act.p, (size_t)e->N * 4, hipMemcpyDeviceToHost, e->stream));
    HIP_TRY(hipStreamSynchronize(e->stream));
  }
  return CRL_OK;
}

int crl_update(crl_engine* e) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (!e->have_transition) return fail(CRL_E_STATE, "crl_update needs a preceding crl_step");
  const crl::Rules R = e->rules();
  const int grid = (e->N + 255) / 256;
  if (e->cfg.table_mode == CRL_TABLE_PER_ENV) {
    if (e->A == 4)
      hipLaunchKernelGGL((crl::k_update_per_env<4>), dim3(grid), dim3(256), 0, e->stream, R, e->ptrs(),
                         e->transition());
    else
      hipLaunchKernelGGL((crl::k_update_per_env<8>), dim3(grid), dim3(256), 0, e->stream, R, e->ptrs(),
                         e->transition());
    HIP_TRY(hipGetLastError());
  } else {
    if (e->A == 4)
      hipLaunchKernelGGL((crl::k_delta<4>), dim3(grid), dim3(256), 0, e->stream, e->Q.p, e->N, e->tr_s.p,
                         e->tr_a.p, e->tr_r.p, e->tr_s2.p, e->tr_done.p, R.lr, R.gamma, R.max_mode,
                         e->key.p, e->delta.p);
    else
      hipLaunchKernelGGL((crl::k_delta<8>), dim3(grid), dim3(256), 0, e->stream, e->Q.p, e->N, e->tr_s.p,
                         e->tr_a.p, e->tr_r.p, e->tr_s2.p, e->tr_done.p, R.lr, R.gamma, R.max_mode,
                         e->key.p, e->delta.p);
    HIP_TRY(hipGetLastError());
    rc = reduce_apply(e, e->Q.p, e->key.p, e->delta.p, e->N);
    if (rc) return rc;
  }
  e->have_transition = false;
  e->t += 1;
  return CRL_OK;
}

int crl_td_update(crl_engine* e, int32_t table, int32_t n, const int32_t* s, const int32_t* a,
                  const float* r, const int32_t* s_next, const uint8_t* done) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (table < 0 || table >= e->n_tables) return fail(CRL_E_RANGE, "table %d outside [0,%d)", table, e->n_tables);
  if (n < 0) return fail(CRL_E_ARG, "negative sample count");
  if (n == 0) return CRL_OK;
  if (!s || !a || !r || !s_next || !done) return fail(CRL_E_ARG, "null transition array");
  for (int i = 0; i < n; ++i) {
    if (s[i] < 0 || (size_t)s[i] >= e->S) return fail(CRL_E_RANGE, "s[%d] = %d outside [0,%zu)", i, s[i], e->S);
    if (s_next[i] < 0 || (size_t)s_next[i] >= e->S)
      return fail(CRL_E_RANGE, "s_next[%d] = %d outside [0,%zu)", i, s_next[i], e->S);
  }
  const size_t nn = (size_t)n;
  hipError_t h = hipSuccess;
  auto acc = [&](hipError_t x) {
    if (h == hipSuccess) h = x;
  };
  acc(e->b_s.ensure(nn));
  acc(e->b_a.ensure(nn));
  acc(e->b_s2.ensure(nn));
  acc(e->b_r.ensure(nn));
  acc(e->b_done.ensure(nn));
  acc(e->key.ensure(nn > (size_t)e->N ? nn : (size_t)e->N));
  acc(e->delta.ensure(nn > (size_t)e->N ? nn : (size_t)e->N));
  if (h != hipSuccess) return fail(CRL_E_ALLOC, "scratch allocation failed: %s", hipGetErrorString(h));
  HIP_TRY(hipMemcpyAsync(e->b_s.p, s, nn * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipMemcpyAsync(e->b_a.p, a, nn * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipMemcpyAsync(e->b_r.p, r, nn * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipMemcpyAsync(e->b_s2.p, s_next, nn * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipMemcpyAsync(e->b_done.p, done, nn, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  float* Q = e->Q.p + (size_t)table * e->K;
  const int grid = (n + 255) / 256;
  if (e->A == 4)
    hipLaunchKernelGGL((crl::k_delta<4>), dim3(grid), dim3(256), 0, e->stream, Q, n, e->b_s.p, e->b_a.p,
                       e->b_r.p, e->b_s2.p, e->b_done.p, e->cfg.lr, e->cfg.gamma, e->cfg.max_mode,
                       e->key.p, e->delta.p);
  else
    hipLaunchKernelGGL((crl::k_delta<8>), dim3(grid), dim3(256), 0, e->stream, Q, n, e->b_s.p, e->b_a.p,
                       e->b_r.p, e->b_s2.p, e->b_done.p, e->cfg.lr, e->cfg.gamma, e->cfg.max_mode,
                       e->key.p, e->delta.p);
  HIP_TRY(hipGetLastError());
  return reduce_apply(e, Q, e->key.p, e->delta.p, n);
}

int crl_run_fused(crl_engine* e, int32_t n_steps) { return run_fused(e, n_steps, false); }

int crl_run_fused_noalloc(crl_engine* e, int32_t n_steps) { return run_fused(e, n_steps, true); }

int crl_get_state(crl_engine* e, int32_t* s, float* reward, uint8_t* done, uint8_t* action,
                  int32_t* ep_step, int32_t* episode) {
  int rc = check_usable(e);
  if (rc) return rc;
  const size_t N = (size_t)e->N;
  if (s) HIP_TRY(hipMemcpyAsync(s, e->s.p, N * 4, hipMemcpyDeviceToHost, e->stream));
  if (reward) HIP_TRY(hipMemcpyAsync(reward, e->reward.p, N * 4, hipMemcpyDeviceToHost, e->stream));
  if (done) HIP_TRY(hipMemcpyAsync(done, e->done.p, N, hipMemcpyDeviceToHost, e->stream));
  if (action) HIP_TRY(hipMemcpyAsync(action, e->action.p, N, hipMemcpyDeviceToHost, e->stream));
  if (ep_step) HIP_TRY(hipMemcpyAsync(ep_step, e->ep_step.p, N * 4, hipMemcpyDeviceToHost, e->stream));
  if (episode) HIP_TRY(hipMemcpyAsync(episode, e->episode.p, N * 4, hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  return check_persist(e);
}

int crl_set_state(crl_engine* e, const int32_t* s, const int32_t* ep_step, const int32_t* episode) {
  int rc = check_engine(e);
  if (rc) return rc;
  rc = clear_persist_failure(e);
  if (rc) return rc;
  const size_t N = (size_t)e->N;
  if (s) {
    for (int i = 0; i < e->N; ++i)
      if (s[i] < 0 || (size_t)s[i] >= e->S) return fail(CRL_E_RANGE, "s[%d] = %d outside [0,%zu)", i, s[i], e->S);
    HIP_TRY(hipMemcpyAsync(e->s.p, s, N * 4, hipMemcpyHostToDevice, e->stream));
  }
  if (ep_step) HIP_TRY(hipMemcpyAsync(e->ep_step.p, ep_step, N * 4, hipMemcpyHostToDevice, e->stream));
  if (episode) HIP_TRY(hipMemcpyAsync(e->episode.p, episode, N * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  e->have_transition = false;
  e->have_actions = false;
  return CRL_OK;
}

int crl_get_episode_stats(crl_engine* e, float* last_return, int32_t* last_length, float* return_sum,
                          int32_t* length_sum) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (!e->cfg.track_returns) return fail(CRL_E_STATE, "the engine was created without track_returns");
  const size_t b = (size_t)e->N * 4;
  if (last_return) HIP_TRY(hipMemcpyAsync(last_return, e->ret_last.p, b, hipMemcpyDeviceToHost, e->stream));
  if (last_length) HIP_TRY(hipMemcpyAsync(last_length, e->len_last.p, b, hipMemcpyDeviceToHost, e->stream));
  if (return_sum) HIP_TRY(hipMemcpyAsync(return_sum, e->ret_sum.p, b, hipMemcpyDeviceToHost, e->stream));
  if (length_sum) HIP_TRY(hipMemcpyAsync(length_sum, e->len_sum.p, b, hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  return CRL_OK;
}

int crl_get_step_count(crl_engine* e, uint64_t* t) {
  if (!e || !t) return fail(CRL_E_ARG, "null argument");
  *t = e->t;
  return CRL_OK;
}

int crl_set_step_count(crl_engine* e, uint64_t t) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  e->t = t;
  return CRL_OK;
}

int crl_q_get_range(crl_engine* e, int32_t first_table, int32_t count, float* out) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (!out) return fail(CRL_E_ARG, "out is null");
  if (first_table < 0 || count < 0 || (int64_t)first_table + count > e->n_tables)
    return fail(CRL_E_RANGE, "table range [%d,%d) outside [0,%d)", first_table, first_table + count, e->n_tables);
  HIP_TRY(hipMemcpyAsync(out, e->Q.p + (size_t)first_table * e->K, (size_t)count * e->K * sizeof(float),
                         hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  return check_persist(e);
}

int crl_q_get(crl_engine* e, int32_t table, float* out) { return crl_q_get_range(e, table, 1, out); }

int crl_q_set(crl_engine* e, int32_t table, const float* in) {
  int rc = check_engine(e);
  if (rc) return rc;
  rc = clear_persist_failure(e);
  if (rc) return rc;
  if (!in) return fail(CRL_E_ARG, "in is null");
  if (table < 0 || table >= e->n_tables) return fail(CRL_E_RANGE, "table %d outside [0,%d)", table, e->n_tables);
  HIP_TRY(hipMemcpyAsync(e->Q.p + (size_t)table * e->K, in, e->K * sizeof(float), hipMemcpyHostToDevice,
                         e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  return CRL_OK;
}

int crl_set_trace(crl_engine* e, int32_t n_envs, int32_t max_steps) {
  int rc = check_engine(e);
  if (rc) return rc;
  if (n_envs < 0 || n_envs > e->N || max_steps < 0) return fail(CRL_E_ARG, "bad trace size");
  HIP_TRY(hipStreamSynchronize(e->stream));
  e->trace_n = 0;
  e->trace_cap = 0;
  e->trace_cursor = 0;
  if (n_envs == 0 || max_steps == 0) return CRL_OK;
  const size_t cells = (size_t)n_envs * max_steps;
  hipError_t h = hipSuccess;
  auto acc = [&](hipError_t x) {
    if (h == hipSuccess) h = x;
  };
  acc(e->trace_s.ensure(cells));
  acc(e->trace_a.ensure(cells));
  acc(e->trace_r.ensure(cells));
  acc(e->trace_d.ensure(cells));
  if (h != hipSuccess) return fail(CRL_E_ALLOC, "trace allocation failed: %s", hipGetErrorString(h));
  e->trace_n = n_envs;
  e->trace_cap = max_steps;
  return CRL_OK;
}

int crl_get_trace(crl_engine* e, int32_t n_steps, int32_t* s_next, uint8_t* action, float* reward,
                  uint8_t* done) {
  int rc = check_usable(e);
  if (rc) return rc;
  if (n_steps < 0 || n_steps > e->trace_cursor)
    return fail(CRL_E_RANGE, "%d steps asked, %d recorded", n_steps, e->trace_cursor);
  const size_t cells = (size_t)n_steps * e->trace_n;
  if (cells == 0) return CRL_OK;
  if (s_next) HIP_TRY(hipMemcpyAsync(s_next, e->trace_s.p, cells * 4, hipMemcpyDeviceToHost, e->stream));
  if (action) HIP_TRY(hipMemcpyAsync(action, e->trace_a.p, cells, hipMemcpyDeviceToHost, e->stream));
  if (reward) HIP_TRY(hipMemcpyAsync(reward, e->trace_r.p, cells * 4, hipMemcpyDeviceToHost, e->stream));
  if (done) HIP_TRY(hipMemcpyAsync(done, e->trace_d.p, cells, hipMemcpyDeviceToHost, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  return check_persist(e);
}

int crl_set_persist_spin_limit(crl_engine* e, int32_t polls) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  if (polls < 1) return fail(CRL_E_ARG, "at least one poll");
  e->persist_spin_limit = polls;
  return CRL_OK;
}

int crl_set_exploration_stream(crl_engine* e, int32_t n_steps, const float* u, const int32_t* a_rand) {
  int rc = check_engine(e);
  if (rc) return rc;
  HIP_TRY(hipStreamSynchronize(e->stream));
  e->sup_n = 0;
  if (!u || n_steps <= 0) return CRL_OK;
  if (!a_rand) return fail(CRL_E_ARG, "a_rand is null");
  const size_t cells = (size_t)n_steps * e->N;
  for (size_t i = 0; i < cells; ++i)
    if (a_rand[i] < 0 || a_rand[i] >= e->A) return fail(CRL_E_RANGE, "a_rand[%zu] = %d outside [0,%d)", i, a_rand[i], e->A);
  hipError_t h = e->u_sup.ensure(cells);
  if (h == hipSuccess) h = e->a_sup.ensure(cells);
  if (h != hipSuccess) return fail(CRL_E_ALLOC, "stream allocation failed: %s", hipGetErrorString(h));
  HIP_TRY(hipMemcpyAsync(e->u_sup.p, u, cells * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipMemcpyAsync(e->a_sup.p, a_rand, cells * 4, hipMemcpyHostToDevice, e->stream));
  HIP_TRY(hipStreamSynchronize(e->stream));
  e->sup_t0 = e->t;
  e->sup_n = n_steps;
  return CRL_OK;
}

int crl_device_ptr(crl_engine* e, int32_t which, void** out) {
  if (!e || !out) return fail(CRL_E_ARG, "null argument");
  switch (which) {
    case CRL_PTR_S: *out = e->s.p; break;
    case CRL_PTR_EP_STEP: *out = e->ep_step.p; break;
    case CRL_PTR_EPISODE: *out = e->episode.p; break;
    case CRL_PTR_REWARD: *out = e->reward.p; break;
    case CRL_PTR_DONE: *out = e->done.p; break;
    case CRL_PTR_ACTION: *out = e->action.p; break;
    case CRL_PTR_Q: *out = e->Q.p; break;
    default: return fail(CRL_E_ARG, "unknown pointer id %d", which);
  }
  return CRL_OK;
}

int crl_fused_kernel_info(crl_engine* e, int32_t n_steps, char* name, size_t name_len, int32_t* grid,
                          int32_t* block, int32_t* lds_bytes) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  if (e->cfg.table_mode == CRL_TABLE_PER_ENV) {
    const FusedPlan p = plan_fused(e, n_steps > 0 ? n_steps : 1 << 20);  // <= 0: a long launch
    if (name && name_len) snprintf(name, name_len, "%s", p.name);
    if (grid) *grid = p.grid;
    if (block) *block = p.block;
    if (lds_bytes) *lds_bytes = (int32_t)p.lds;
  } else {
    const PersistPlan pp = plan_persist(e, n_steps > 0 ? n_steps : 1 << 20);
    if (pp.ok) {
      if (name && name_len) snprintf(name, name_len, "k_shared_persist<%d,%d%s>", e->A, pp.lds_map ? 1 : 2, pp.fold ? ",folded" : "");
      if (grid) *grid = pp.grid;
      if (block) *block = 256;
      if (lds_bytes) *lds_bytes = (int32_t)pp.lds;
      return CRL_OK;
    }
    if (name && name_len) snprintf(name, name_len, "k_shared_act+k_reduce_owners");
    if (grid) *grid = (e->N + 255) / 256;
    if (block) *block = 256;
    if (lds_bytes) *lds_bytes = e->map_words * 4;
  }
  return CRL_OK;
}

int crl_fused_plan_for_config(const crl_config* cfg, int32_t n_steps, char* name, size_t name_len,
                              int32_t* grid, int32_t* block, int32_t* lds_bytes) {
  int rc = crl::validate_config(cfg, crl::last_error());
  if (rc != CRL_OK) return rc;
  if (cfg->table_mode != CRL_TABLE_PER_ENV) return fail(CRL_E_ARG, "only per-env tables have a fused launch plan");
  crl_engine shell;  // sizes only: nothing is allocated and no device is touched
  set_geometry(&shell, *cfg);
  const FusedPlan p = plan_fused(&shell, n_steps > 0 ? n_steps : 1 << 20);
  if (name && name_len) snprintf(name, name_len, "%s", p.name);
  if (grid) *grid = p.grid;
  if (block) *block = p.block;
  if (lds_bytes) *lds_bytes = (int32_t)p.lds;
  if (p.grid < 1 || p.block < 64 || p.block > 1024 || p.lds > kLdsPerWorkgroup)
    return fail(CRL_E_STATE, "launch plan %s: grid %d, block %d, %zu bytes of LDS", p.name, p.grid, p.block, p.lds);
  return CRL_OK;
}

// Diagnostics: arms (or disarms) the phase clocks of the one-launch shared-table kernel.
// Armed, the instantiation that reads the shader clock eight times per step runs.
int crl_set_persist_clocks(crl_engine* e, int32_t on) {
  if (!e) return fail(CRL_E_ARG, "null engine");
  e->persist_clocks = on != 0;
  return CRL_OK;
}

// Diagnostics: what the last one-launch shared-table launch that ran with the clocks armed
// left behind (layout: include/crl.h); at most n_words 64-bit words are copied.
int crl_get_persist_clocks(crl_engine* e, uint64_t* out, size_t n_words) {
  int rc = check_engine(e);
  if (rc) return rc;
  if (!out) return fail(CRL_E_ARG, "out is null");
  if (!e->pdiag.p) return fail(CRL_E_STATE, "this engine has no shared table");
  HIP_TRY(hipStreamSynchronize(e->stream));
  rc = check_persist(e);
  if (rc) return rc;
  const size_t n = std::min<size_t>(n_words, crl::kPersistClockWords);
  HIP_TRY(hipMemcpy(out, e->pdiag.p + 1, n * sizeof(uint64_t), hipMemcpyDeviceToHost));
  return CRL_OK;
}

// Measurement helper: nanoseconds per barrier over `n_groups` co-resident workgroups
// built from device-scope loads and stores (pattern: see k_probe_barrier).
int crl_probe_barrier(int pattern, int n_groups, int rounds, double* ns_per_barrier) {
  if (pattern < 0 || pattern > 2 || n_groups < 1 || n_groups > crl::kPersistMaxGroups || rounds < 1 || !ns_per_barrier)
    return fail(CRL_E_ARG, "pattern 0..2, 1..%d workgroups, rounds >= 1", crl::kPersistMaxGroups);
  const size_t words = (size_t)(17 + crl::kPersistMaxGroups) * crl::kProbeLine;
  DevBuf<unsigned> mem;
  DevBuf<unsigned long long> out;
  if (mem.alloc(words) != hipSuccess || out.alloc(2) != hipSuccess) return fail(CRL_E_ALLOC, "probe allocation failed");
  HIP_TRY(hipMemset(mem.p, 0, words * sizeof(unsigned)));
  HIP_TRY(hipMemset(out.p, 0, 2 * sizeof(unsigned long long)));
  unsigned* m = mem.p;
  unsigned long long* o = out.p;
  void* args[] = {&m, &rounds, &o};
  const void* kern = pattern == 0   ? reinterpret_cast<const void*>(&crl::k_probe_barrier<0>)
                     : pattern == 1 ? reinterpret_cast<const void*>(&crl::k_probe_barrier<1>)
                                    : reinterpret_cast<const void*>(&crl::k_probe_barrier<2>);
  // co-resident or refused: the workgroups wait for each other
  HIP_TRY(hipLaunchCooperativeKernel(kern, dim3(n_groups), dim3(256), args, 0, nullptr));
  HIP_TRY(hipDeviceSynchronize());
  unsigned long long h[2];
  HIP_TRY(hipMemcpy(h, out.p, sizeof h, hipMemcpyDeviceToHost));
  if (h[1]) return fail(CRL_E_DEVICE, "%llu workgroups gave up waiting", h[1]);
  *ns_per_barrier = (double)h[0] * 10.0 / rounds;  // 100 MHz ticks
  return CRL_OK;
}


int crl_probe_copy(size_t n_bytes, int repeats) {
  if (n_bytes == 0 || n_bytes % 16 != 0 || repeats < 1) return fail(CRL_E_ARG, "n_bytes must be a positive multiple of 16");
  DevBuf<uint8_t> src, dst;
  if (src.alloc(n_bytes) != hipSuccess || dst.alloc(n_bytes) != hipSuccess)
    return fail(CRL_E_ALLOC, "probe allocation failed");
  HIP_TRY(hipMemset(src.p, 1, n_bytes));
  HIP_TRY(hipMemset(dst.p, 0, n_bytes));
  const size_t n16 = n_bytes / 16;
  for (int i = 0; i < repeats; ++i)
    hipLaunchKernelGGL(crl::k_probe_copy, dim3(256 * 16), dim3(256), 0, nullptr,
                       reinterpret_cast<const uint4*>(src.p), reinterpret_cast<uint4*>(dst.p), n16);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipDeviceSynchronize());
  // the copy arrived: both ends of the destination hold the source's pattern
  uint8_t ends[2][256];
  const size_t tail = n_bytes >= sizeof ends[0] ? n_bytes - sizeof ends[0] : 0;
  const size_t len = n_bytes >= sizeof ends[0] ? sizeof ends[0] : n_bytes;
  HIP_TRY(hipMemcpy(ends[0], dst.p, len, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(ends[1], dst.p + tail, len, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < len; ++i)
    if (ends[0][i] != 1 || ends[1][i] != 1) return fail(CRL_E_DEVICE, "copy kernel left byte %zu unwritten", i);
  return CRL_OK;
}

}  // extern "C"
