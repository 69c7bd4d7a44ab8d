/*
 * crl.h - C ABI of the MI355X (gfx950) batched grid-world + tabular Q-learning engine.
 *
 * Everything here is `extern "C"`, plain pointers and sizes.  Every function
 * returns an int status (CRL_OK or a negative CRL_E_* code) unless stated;
 * `crl_last_error()` gives the text of the calling thread's last failure.
 * Nothing throws across this boundary.  Host buffers belong to the caller,
 * device buffers to the engine.  Calls on one engine must be serialised by
 * the caller; there is no CPU fallback: without a usable HIP device
 * `crl_create` fails with CRL_E_DEVICE.
 *
 * Built for MI355X only: the launch plans assume its 256 compute units, 160 KB
 * of LDS per workgroup and 256 MB last-level cache as compile-time constants
 * (they are not read from hipDeviceProp_t); on another gfx950 part results stay
 * the same and only the tuning is off.
 *
 * Citations name the file:line of life423/CudaRL-Arena that the entry point
 * replaces.  State index is s = y*W + x and the table layout is
 * Q[s*A + a], fp32 (src/kernels.cu:96, src/q_learning.cu:196).
 *
 * Actions (src/kernels.cu:15-23): 0 = up (dy-1), 1 = right (dx+1),
 * 2 = down (dy+1), 3 = left (dx-1); any other value is "no move".  With
 * n_actions == 8 the diagonals follow: 4 = up-right, 5 = down-right,
 * 6 = down-left, 7 = up-left.
 */
#ifndef CRL_H
#define CRL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CRL_VERSION "0.1.0" /* src/python_bindings.cpp:24 */

/* status codes */
enum {
  CRL_OK = 0,
  CRL_E_ARG = -1,      /* bad argument / inconsistent sizes               */
  CRL_E_DEVICE = -2,   /* no HIP device, or a HIP call failed             */
  CRL_E_ALLOC = -3,    /* device or host allocation failed                */
  CRL_E_STATE = -4,    /* call not valid in the engine's current state    */
  CRL_E_RANGE = -5     /* index out of range                              */
};

/* cell classes; thresholds on the reference's float grid are
 * FREE [0,0.99), GOAL >= 0.99, TRAP (-1,0), WALL <= -1 (src/kernels.cu:30-63) */
enum { CRL_CELL_FREE = 0, CRL_CELL_GOAL = 1, CRL_CELL_TRAP = 2, CRL_CELL_WALL = 3 };

enum { CRL_TABLE_PER_ENV = 0, CRL_TABLE_SHARED = 1 };
enum { CRL_MAP_PER_ENV = 0, CRL_MAP_SHARED = 1 };

/* max over the next row: TRUE_MAX follows src/gpu/kernels.cu:35-45,
 * ZERO_FLOOR follows src/kernels.cu:101-110 (max seeded with 0.0f). */
enum { CRL_MAX_TRUE = 0, CRL_MAX_ZERO_FLOOR = 1 };

/* goal test: TARGET follows src/kernels.cu:50-58 (class of the in-bounds
 * target cell), RESULT follows src/environment.cu:43 (class of the cell the
 * agent stands on after the move, so an out-of-bounds bump on the goal
 * re-fires it). */
enum { CRL_GOAL_ON_TARGET = 0, CRL_GOAL_ON_RESULT = 1 };

/* exploration schedules (src/train.py:100-108,140-141) */
enum {
  CRL_EPS_FIXED = 0,            /* eps0 for ever                                   */
  CRL_EPS_STEP_MULT = 1,        /* eps0 * decay^t, t = global step (the reference) */
  CRL_EPS_EPISODE_MULT = 2,     /* eps0 * decay^episode, per env                   */
  CRL_EPS_EPISODE_LINEAR = 3    /* eps0 -> eps_end linearly over eps_span episodes */
};

/* reward_flags bits */
enum {
  CRL_REWARD_CELLS = 1,      /* a per-cell fp32 array gives the goal / trap rewards   */
  CRL_REWARD_BASE_CELLS = 2  /* ... and also the plain-step reward (cell stood on)    */
};

typedef struct crl_config {
  uint32_t struct_size;  /* sizeof(crl_config), checked                            */
  int32_t n_envs;        /* N >= 1                                                 */
  int32_t width, height; /* W, H >= 1; S = W*H                                      */
  int32_t n_actions;     /* A: 4 or 8                                              */
  int32_t table_mode;    /* CRL_TABLE_*                                            */
  int32_t map_mode;      /* CRL_MAP_*                                              */
  int32_t max_mode;      /* CRL_MAX_*                                              */
  int32_t goal_mode;     /* CRL_GOAL_*                                             */
  int32_t auto_reset;    /* 1: an env that is done or has used episode_len steps
                            restarts from its start cell; 0: done is sticky
                            (src/environment.cu:44-46 never clears it)             */
  int32_t episode_len;   /* T; 0 = no limit                                        */
  float lr, gamma;       /* src/q_learning.cuh:18-19                               */
  float step_reward;     /* -0.01f (src/kernels.cu:46)                             */
  float goal_reward;     /*  1.0f  (src/kernels.cu:56)                             */
  float trap_reward;     /* bump penalty of a TRAP cell when no cell array is set   */
  int32_t reward_flags;  /* CRL_REWARD_* bits                                      */
  int32_t eps_mode;      /* CRL_EPS_*                                              */
  float eps0, eps_decay, eps_end;
  int32_t eps_span;      /* table length for the STEP/EPISODE schedules            */
  int32_t max_episodes;  /* > 0: an env stops stepping once it has finished this
                            many episodes (the `for episode in range(num_episodes)`
                            of src/train.py:191); 0 = no budget                    */
  int32_t track_returns; /* 1: keep per-env episode return / length accumulators
                            on the device (src/train.py:205-226)                   */
  uint64_t seed;         /* Philox4x32-10 key                                      */
} crl_config;

typedef struct crl_engine crl_engine;

/* -- life cycle ---------------------------------------------------------- */

const char* crl_last_error(void);
const char* crl_version(void);
/* number of HIP devices, or a negative status */
int crl_device_count(void);

/* Replaces the constructors Environment::Environment (src/environment.cu:50-77)
 * and CudaQLearning::CudaQLearning (src/q_learning.cu:6-94): allocates the SoA
 * state, the map and the zero-initialised table(s) on device `device`.  All
 * envs start on cell 0 of an all-FREE map until crl_set_maps is called. */
int crl_create(const crl_config* cfg, int device, crl_engine** out);
/* Replaces ~Environment / ~CudaQLearning (src/environment.cu:79-100,
 * src/q_learning.cu:96-106).  NULL is allowed. */
int crl_destroy(crl_engine* e);
/* Use `hip_stream` (a hipStream_t, NULL = the null stream) for all later work. */
int crl_set_stream(crl_engine* e, void* hip_stream);
int crl_sync(crl_engine* e);
/* Tuning (no reference counterpart): how many envs crl_run_fused keeps in
 * flight at once for per-env tables; the rest follow in turn inside the same
 * launch.  0 = automatic (as many as keep the tables in the last-level cache).
 * Results do not depend on it. */
int crl_set_resident_envs(crl_engine* e, int32_t n_envs);
/* Tuning (no reference counterpart): kernel of crl_run_fused.  0 = automatic.
 * Per-env tables: 1 = plain (every wave steps envs against tables in HBM),
 * 2 = hybrid (the last wave of each workgroup steps envs whose whole tables it holds
 * in LDS; used only when 32 tables fit; automatic picks it for launches of at
 * least 64 steps).  Shared table: 1 = two launches per step; 2 = all steps of a
 * call in one launch whose 256 workgroups exchange block sums and table values
 * through device-scope loads and stores (needs every workgroup resident at once:
 * at most 65,536 envs and 16,384 table entries, else two launches per step);
 * automatic picks the one launch for calls of at least 4 steps.
 * Results do not depend on it. */
int crl_set_fused_variant(crl_engine* e, int32_t variant);
/* How the last hybrid crl_run_fused split the envs between its two kinds of
 * workers (tables in HBM / tables in LDS); both 0 if the plain kernel ran. */
int crl_get_fused_split(crl_engine* e, uint32_t* hbm_envs, uint32_t* lds_envs);

/* -- maps ------------------------------------------------------------------ */

/* Replaces Environment::initializeGrid + the H2D grid copy
 * (src/environment.cu:60-74,138-147).  cell_class: n_maps*S bytes of CRL_CELL_*
 * (n_maps = N, or 1 when map_mode is SHARED); start: N cell indices (NULL keeps
 * the current ones); cell_reward: n_maps*S floats, required iff reward_flags has
 * CRL_REWARD_CELLS.  Also resets every env (as crl_reset(e,0,N)). */
int crl_set_maps(crl_engine* e, const uint8_t* cell_class, const int32_t* start,
                 const float* cell_reward);
/* Edit one cell; gives EnvironmentBridge::addObstacle/setGoal/addTrap
 * (src/environment_bridge.cu:53-78, print-only upstream) an effect. */
int crl_set_cell(crl_engine* e, int32_t map_index, int32_t cell, int32_t cell_class,
                 float cell_reward);
/* Classify the reference's float grid (thresholds of src/kernels.cu:30-63):
 * out_class[i] in CRL_CELL_*, out_reward[i] = 1.0f for GOAL, v for TRAP,
 * step_reward otherwise.  Host only. */
int crl_classify_grid(const float* grid, size_t n, float step_reward, uint8_t* out_class,
                      float* out_reward);

/* -- the hot path ---------------------------------------------------------- */

/* Environment::reset (src/environment.cu:102-111; kernel :6-14): envs
 * [first, first+count) go to their start cell, reward 0, done false,
 * episode step 0.  The episode counter is not changed. */
int crl_reset(crl_engine* e, int32_t first, int32_t count);

/* Environment::step (src/environment.cu:113-125) with the wall / trap / goal
 * rules of step_environment_kernel (src/kernels.cu:13-66), for all N envs.
 * `actions` = N host int32 (NULL: use the actions the last crl_select left on
 * the device).  Records the transition (s, a, r, s', done) for crl_update. */
int crl_step(crl_engine* e, const int32_t* actions);

/* Epsilon-greedy selection (src/train.py:100-108) with the greedy branch of
 * CudaQLearning::get_best_action (src/q_learning.cu:191-209: lowest index wins
 * ties).  The uniforms come from Philox4x32-10 keyed (seed; env, step) unless an
 * exploration stream was supplied.  actions_out: N host int32 or NULL. */
int crl_select(crl_engine* e, int32_t* actions_out);

/* TD update of the transition recorded by the last crl_step
 * (src/gpu/kernels.cu:7-54); advances the global step counter by one. */
int crl_update(crl_engine* e);

/* CudaQLearning::update_batch (src/q_learning.cu:108-174): n explicit
 * transitions on table `table` (0 for a shared table, the env index
 * otherwise).  All reads see the table as it was before the call; deltas that
 * hit the same (s,a) are summed in sample order and then applied.  Host arrays.
 * States outside the table are refused (CRL_E_RANGE); a sample whose action is
 * outside [0, n_actions) changes nothing, as a step with such an action moves
 * nothing (src/kernels.cu:15-23). */
int crl_td_update(crl_engine* e, int32_t table, int32_t n, const int32_t* s, const int32_t* a,
                  const float* r, const int32_t* s_next, const uint8_t* done);

/* n_steps of select -> step -> update for every env, fused on the device
 * (the loop body of src/train.py:198-222).  Same results as n_steps rounds of
 * crl_select; crl_step(NULL); crl_update. */
int crl_run_fused(crl_engine* e, int32_t n_steps);

/* crl_run_fused for callers that cannot allocate device memory (tight serving
 * loops, harnesses that forbid hipMalloc): no counterpart in the reference.
 * Same results as crl_run_fused, but its scratch - the ticket counters of the
 * per-env kernels, the hand-off cells of the shared table's ordered reduction,
 * the exchange buffers of the one-launch shared-table kernel - lives in a
 * static device array of 10 MB + 4 KB that each GPU the library runs on holds
 * until the process ends, and the call allocates and frees nothing (device or
 * host).  CRL_E_RANGE if the engine's ordered reduction needs more hand-off cells
 * than the array holds (65,536 envs on a 64x64x4 table need 4 MB with two launches
 * per step, 9.7 MB of exchange buffers in the one-launch kernel; an engine whose
 * one-launch buffers do not fit takes two launches per step).  All engines on one GPU share that GPU's
 * array: calls that overlap in time on one GPU (different streams or threads)
 * race; calls in stream order do not. */
int crl_run_fused_noalloc(crl_engine* e, int32_t n_steps);

/* Environment getters (src/environment.h:26-37) for all envs; any pointer may
 * be NULL.  s = cell the env acts from next, reward/done/action = last step. */
int crl_get_state(crl_engine* e, int32_t* s, float* reward, uint8_t* done, uint8_t* action,
                  int32_t* ep_step, int32_t* episode);
/* Restore a saved state (checkpoint / resume; no reference counterpart beyond
 * get/set_q_table).  Any pointer may be NULL. */
int crl_set_state(crl_engine* e, const int32_t* s, const int32_t* ep_step,
                  const int32_t* episode);
/* Episode statistics (needs track_returns): return and length of the last
 * finished episode of every env, and their sums over all finished episodes
 * (the number of finished episodes is `episode` of crl_get_state).  Any pointer
 * may be NULL.  Replaces the episode_rewards / episode_lengths lists of
 * src/train.py:186-226. */
int crl_get_episode_stats(crl_engine* e, float* last_return, int32_t* last_length,
                          float* return_sum, int32_t* length_sum);
/* global step counter t (number of updates so far) */
int crl_get_step_count(crl_engine* e, uint64_t* t);
int crl_set_step_count(crl_engine* e, uint64_t t);

/* CudaQLearning::get_q_table / set_q_table (src/q_learning.cu:176-189):
 * S*A floats of table `table`. */
int crl_q_get(crl_engine* e, int32_t table, float* out);
int crl_q_set(crl_engine* e, int32_t table, const float* in);
/* several consecutive tables in one copy */
int crl_q_get_range(crl_engine* e, int32_t first_table, int32_t count, float* out);

/* -- test hooks ------------------------------------------------------------ */

/* Record (s', action, reward, done) of envs [0, n_envs) for the next
 * `max_steps` steps run by crl_run_fused / crl_step.  n_envs = 0 turns it off. */
int crl_set_trace(crl_engine* e, int32_t n_envs, int32_t max_steps);
/* Copy out `n_steps` recorded steps, arrays [n_steps][n_trace_envs]. */
int crl_get_trace(crl_engine* e, int32_t n_steps, int32_t* s_next, uint8_t* action,
                  float* reward, uint8_t* done);
/* Supply the exploration stream instead of Philox: u[n_steps][N] in [0,1) and
 * a_rand[n_steps][N] in [0,A), consumed by steps t0 .. t0+n_steps-1 where t0 is
 * the step counter at the time of this call.  NULL u removes it. */
int crl_set_exploration_stream(crl_engine* e, int32_t n_steps, const float* u,
                               const int32_t* a_rand);

/* How many polls a thread of the one-launch shared-table kernel waits for its
 * peers' data before it gives up (default 2^20, a few hundred milliseconds).  A
 * workgroup that gives up sets a word that the others see and leave on, and that
 * makes later launches of the kernel return at once; the next call that
 * synchronises (crl_sync, crl_get_state, crl_q_get, crl_get_trace,
 * crl_get_episode_stats) fails with CRL_E_DEVICE, once.  The engine's state and
 * table are not valid from then on: every call that works on them fails with
 * CRL_E_STATE until the caller sets them again (crl_reset, crl_set_state or
 * crl_q_set).  With a limit of 1 every workgroup leaves at its first unanswered
 * poll: how the tests exercise that path without a kernel that hangs. */
int crl_set_persist_spin_limit(crl_engine* e, int32_t polls);

/* raw device pointers of the SoA state for zero-copy consumers; index with
 * CRL_PTR_*.  Valid until crl_destroy.  What they point at is the engine's as
 * of the last call on its stream: call crl_sync first (which also reports a
 * one-launch kernel that gave up). */
enum {
  CRL_PTR_S = 0, CRL_PTR_EP_STEP = 1, CRL_PTR_EPISODE = 2, CRL_PTR_REWARD = 3,
  CRL_PTR_DONE = 4, CRL_PTR_ACTION = 5, CRL_PTR_Q = 6, CRL_PTR_COUNT = 7
};
int crl_device_ptr(crl_engine* e, int32_t which, void** out);

/* name and launch geometry of the kernel crl_run_fused(e, n_steps) would use for
 * this engine (the plan depends on the launch length: short launches keep every
 * table in HBM and every env in flight).  n_steps <= 0 asks for the plan of a
 * long launch. */
int crl_fused_kernel_info(crl_engine* e, int32_t n_steps, char* name, size_t name_len,
                          int32_t* grid, int32_t* block, int32_t* lds_bytes);

/* The same for an engine that crl_create(cfg) would make, without making one
 * (host only, needs no device): CRL_E_STATE if the plan does not fit the device's
 * limits (160 KB of LDS per workgroup).  Per-env tables only. */
int crl_fused_plan_for_config(const crl_config* cfg, int32_t n_steps, char* name, size_t name_len,
                              int32_t* grid, int32_t* block, int32_t* lds_bytes);

/* -- diagnostics (no reference counterpart; not part of the drop-in surface) -- */

/* One launch of a plain copy kernel `k_probe_copy` moving n_bytes from one device
 * buffer to another, so that hardware traffic counters can be scaled by a launch
 * of known size. */
int crl_probe_copy(size_t n_bytes, int repeats);

/* Phase clocks of the one-launch shared-table kernel.  crl_set_persist_clocks(e, 1)
 * makes later launches run the instantiation that reads the shader clock between
 * the phases of every step (off by default: the product kernel carries no clocks);
 * crl_get_persist_clocks copies what the last such launch left, at most n_words
 * 64-bit words of CRL_PERSIST_CLOCK_WORDS:
 *   [0..7]   first workgroup: shader clocks per phase, summed over the steps
 *   [8..9]   first workgroup, thread 0: polls of the table wait / of the cells wait
 *   [10..19] the same ten words of the last workgroup
 *   [20 + 8 w + p]  100 MHz wall clock at which workgroup w passed the mark that ends
 *            phase p in the middle step of the launch (w < 256)
 * Phases: 0 what a step needs that does not depend on the table, 1 wait for the table,
 * 2 select / move / delta, 3 ordered block sums + cells, 4 clearing the owner's tile and
 * waiting for the cells' acknowledgement, 5 wait for the others' cells, 6 tile, sums,
 * publish, 7 loop overhead. */
#define CRL_PERSIST_CLOCK_WORDS (20 + 8 * 256)
int crl_set_persist_clocks(crl_engine* e, int32_t on);
int crl_get_persist_clocks(crl_engine* e, uint64_t* out, size_t n_words);
/* Nanoseconds per barrier over n_groups (<= 256) co-resident workgroups that meet
 * through device-scope loads and stores.  pattern 0: packed flags, all polled by
 * everybody; 1: one flag per 128-byte line; 2: a tree in which every word has one
 * writer and one reader. */
int crl_probe_barrier(int pattern, int n_groups, int rounds, double* ns_per_barrier);

/* -- host-side helpers (no device needed) ----------------------------------- */

/* Philox4x32-10 (Salmon et al. 2011), exposed for tests. */
void crl_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* the two exploration draws of (seed, env, step t): u in [0,1), a in [0,A) */
void crl_explore_draw(uint64_t seed, uint32_t env, uint64_t t, int32_t n_actions, float* u,
                      int32_t* a_rand);
/* epsilon table the engine would build for cfg (length written to *len, at
 * most cap entries copied) */
int crl_eps_table(const crl_config* cfg, float* out, int32_t cap, int32_t* len);

/* Synthetic maps (no reference counterpart: src/environment.cu:140 seeds from
 * the wall clock).  Cells are WALL with probability p_wall, then TRAP with
 * probability p_trap among the rest; one GOAL per map and N start cells drawn
 * uniformly among the FREE cells.  n_maps = 1 gives a shared map with n_envs
 * starts.  All draws are Philox4x32-10 from `seed`. */
int crl_gen_maps_bernoulli(uint64_t seed, int32_t n_maps, int32_t n_envs, int32_t width,
                           int32_t height, float p_wall, float p_trap, uint8_t* cell_class,
                           int32_t* start);
/* Value-noise maps (lattice pitch `pitch`, smoothstep-bilinear): the
 * `wall_frac` highest-valued cells are WALL; cell_reward = sigma * N(0,1) with
 * goal_bonus added on the GOAL cell. */
int crl_gen_maps_noise(uint64_t seed, int32_t n_maps, int32_t width, int32_t height,
                       int32_t pitch, float wall_frac, float sigma, float goal_bonus,
                       uint8_t* cell_class, int32_t* start, float* cell_reward);

#ifdef __cplusplus
}
#endif
#endif /* CRL_H */
