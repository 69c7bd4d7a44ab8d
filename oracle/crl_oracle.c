/*
 * crl_oracle.c - CPU restatement of the CudaRL-Arena hot path.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP engine is compared
 * against; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load it.  The product never calls it.
 *
 * Scalar C, one env at a time, no vectorisation tricks.  Each function cites
 * the file:line of life423/CudaRL-Arena it follows.  Compile with
 * -ffp-contract=off: the two fused multiply-adds of the TD update are written
 * as explicit fmaf so that every compiler produces the same bits.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   orc_reset_xy, orc_step_e1     the Catch2 cases of tests/test_environment.cpp
 *   orc_step_e2, orc_classify     no reference test exists: pinned by the
 *                                 invariants of src/kernels.cu:13-66 on a
 *                                 brute-forced grid holding every cell class and
 *                                 the threshold edge values, and by reducing to
 *                                 orc_step_e1 on obstacle-free grids
 *   orc_step_cls                  equality with orc_step_e2 on classified grids
 *   orc_argmax                    src/q_learning.cu:191-209 tie rule, numpy argmax
 *   orc_td_*                      closed forms (geometric series), float64 numpy
 *                                 restatement of src/train.py:127-138
 *   orc_philox4x32_10             Random123 known-answer vectors
 *   orc_run + eps schedule        training.log:24931-24953 (returns -5.00 / -10.00,
 *                                 epsilon 0.082, 0.007, 0.001)
 *   ordered reduction (shared)    defined here, not by the reference: brute force
 *                                 of the definition key by key, and (up to 256
 *                                 samples) a dictionary-of-lists summation
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* same field order as the engine's configuration block so that one ctypes
 * structure serves both; declared independently on purpose */
typedef struct orc_config {
  uint32_t struct_size;
  int32_t n_envs;
  int32_t width, height;
  int32_t n_actions;
  int32_t table_mode; /* 0 per env, 1 shared */
  int32_t map_mode;   /* 0 per env, 1 shared */
  int32_t max_mode;   /* 0 true max, 1 zero floor */
  int32_t goal_mode;  /* 0 on target cell, 1 on resulting cell */
  int32_t auto_reset;
  int32_t episode_len;
  float lr, gamma;
  float step_reward, goal_reward, trap_reward;
  int32_t reward_flags; /* 1 cell array for goal/trap, 2 also for the base */
  int32_t eps_mode;     /* 0 fixed, 1 step mult, 2 episode mult, 3 episode linear */
  float eps0, eps_decay, eps_end;
  int32_t eps_span;
  int32_t max_episodes;  /* > 0: an env stops after this many episodes (src/train.py:191) */
  int32_t track_returns; /* informational here: the stats arrays are passed explicitly */
  uint64_t seed;
} orc_config;

enum { FREE = 0, GOAL = 1, TRAP = 2, WALL = 3 };

/* ---- Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11) ------------------- */

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int round = 0; round < 10; ++round) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Exploration draws of (seed, env, step t).  Counter = (env, stream 0,
 * block lo, block hi) with block = t >> 1; even steps take words 0,1 and odd
 * steps words 2,3.  u = top 24 bits / 2^24; a = (word * A) >> 32. */
void orc_explore_draw(uint64_t seed, uint32_t env, uint64_t t, int32_t A, float* u,
                      int32_t* a_rand) {
  uint64_t blk = t >> 1;
  uint32_t ctr[4] = {env, 0u, (uint32_t)blk, (uint32_t)(blk >> 32)};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t w[4];
  orc_philox4x32_10(ctr, key, w);
  uint32_t w0 = (t & 1) ? w[2] : w[0];
  uint32_t w1 = (t & 1) ? w[3] : w[1];
  *u = (float)(w0 >> 8) * (1.0f / 16777216.0f);
  *a_rand = (int32_t)(((uint64_t)w1 * (uint32_t)A) >> 32);
}

/* ---- E0: reset (src/kernels.cu:3-11, src/environment.cu:6-14) ------------ */

void orc_reset_xy(int W, int H, int* x, int* y, float* reward, int* done) {
  *x = W / 2;
  *y = H / 2;
  *reward = 0.0f;
  *done = 0;
}

static void action_delta(int action, int* dx, int* dy) {
  *dx = 0;
  *dy = 0;
  switch (action) { /* src/kernels.cu:18-23; 4..7 are this build's diagonals */
    case 0: *dy = -1; break;
    case 1: *dx = 1; break;
    case 2: *dy = 1; break;
    case 3: *dx = -1; break;
    case 4: *dx = 1; *dy = -1; break;
    case 5: *dx = 1; *dy = 1; break;
    case 6: *dx = -1; *dy = 1; break;
    case 7: *dx = -1; *dy = -1; break;
    default: break;
  }
}

/* ---- E1: step without obstacles (src/environment.cu:17-48) --------------- */

void orc_step_e1(int W, int H, int* x, int* y, float* reward, int* done, int action) {
  int dx = 0, dy = 0;
  if (action >= 0 && action <= 3) action_delta(action, &dx, &dy);
  int nx = *x + dx, ny = *y + dy;
  if (nx >= 0 && nx < W && ny >= 0 && ny < H) {
    *x = nx;
    *y = ny;
  }
  *reward = -0.01f;
  if (*x == W - 1 && *y == 0) {
    *reward = 1.0f;
    *done = 1; /* never cleared: sticky */
  }
}

/* ---- E2: step on a float grid (src/kernels.cu:13-66) --------------------- */

void orc_step_e2(const float* grid, int W, int H, int* x, int* y, float* reward, int* done,
                 int action) {
  int dx = 0, dy = 0;
  if (action >= 0 && action <= 3) action_delta(action, &dx, &dy);
  int nx = *x + dx, ny = *y + dy;
  int in = nx >= 0 && nx < W && ny >= 0 && ny < H;
  int idx = ny * W + nx;
  int obstacle = 0;
  if (in) obstacle = grid[idx] < 0.0f; /* :34 */
  if (in && !obstacle) {                /* :38-43 */
    *x = nx;
    *y = ny;
  }
  *reward = -0.01f; /* :46 */
  if (in) {
    float v = grid[idx];
    if (v >= 0.99f) { /* :55-58 */
      *reward = 1.0f;
      *done = 1;
    } else if (v < 0.0f && v > -1.0f) { /* :60-62 */
      *reward = v;
    }
  }
}

/* cell class of a float cell value, thresholds of src/kernels.cu:34,55,60 */
uint8_t orc_classify(float v) {
  if (v >= 0.99f) return GOAL;
  if (v < 0.0f && v > -1.0f) return TRAP;
  if (v < 0.0f) return WALL; /* v <= -1 */
  return FREE;               /* [0, 0.99), and NaN: no comparison holds */
}

/* ---- generalised step on cell classes ------------------------------------ */
/* cls / cr describe ONE map of S cells.  Returns the hit flag (goal reached
 * in this step); *s is replaced by the cell after the move. */
int orc_step_cls(const orc_config* c, const uint8_t* cls, const float* cr, int32_t* s,
                 int action, float* reward) {
  const int W = c->width, H = c->height;
  int x = *s % W, y = *s / W;
  int dx = 0, dy = 0;
  if (action >= 0 && action < c->n_actions) action_delta(action, &dx, &dy);
  int nx = x + dx, ny = y + dy;
  int in = nx >= 0 && nx < W && ny >= 0 && ny < H;
  int tgt = ny * W + nx;
  int k = in ? cls[tgt] : FREE;
  int moved = in && k < TRAP; /* v < 0 blocks: traps and walls */
  int s2 = moved ? tgt : *s;
  const int cells = (c->reward_flags & 1) != 0;
  float r = (cells && (c->reward_flags & 2)) ? cr[s2] : c->step_reward;
  int hit = 0;
  if (c->goal_mode == 0) {
    if (in) {
      if (k == GOAL) {
        r = cells ? cr[tgt] : c->goal_reward;
        hit = 1;
      } else if (k == TRAP) {
        r = cells ? cr[tgt] : c->trap_reward;
      }
    }
  } else { /* goal test on the resulting cell (src/environment.cu:43) */
    if (in && k == TRAP) r = cells ? cr[tgt] : c->trap_reward;
    if (cls[s2] == GOAL) {
      r = cells ? cr[s2] : c->goal_reward;
      hit = 1;
    }
  }
  *s = s2;
  *reward = r;
  return hit;
}

/* ---- S2: greedy argmax (src/q_learning.cu:191-209) ----------------------- */

int orc_argmax(const float* row, int A) {
  int best = 0;
  float bv = row[0];
  for (int a = 1; a < A; ++a) {
    if (row[a] > bv) {
      bv = row[a];
      best = a;
    }
  }
  return best;
}

/* ---- S1: epsilon-greedy (src/train.py:100-108) --------------------------- */

int orc_select(const float* row, int A, float eps, float u, int a_rand) {
  if (u < eps) return a_rand;
  return orc_argmax(row, A);
}

/* ---- Q1 / Q2: TD target and update --------------------------------------- */

/* max over the next row; mode 0 = true max (src/gpu/kernels.cu:35-45),
 * mode 1 = seeded with 0.0f (src/kernels.cu:101-110) */
float orc_next_max(const float* next_row, int A, int done, int mode) {
  float m = 0.0f;
  if (!done) {
    for (int a = 0; a < A; ++a) {
      float q = next_row[a];
      if (mode == 0)
        m = (a == 0) ? q : fmaxf(m, q);
      else
        m = fmaxf(m, q);
    }
  }
  return m;
}

/* new value of Q[s,a] (src/gpu/kernels.cu:47-52), with the two contractions a
 * GPU compiler makes written out */
float orc_td_value(float q, float r, float m, float lr, float gamma) {
  float target = fmaf(gamma, m, r);
  return fmaf(lr, target - q, q);
}

/* delta of one sample for the summed (batch / shared table) form */
float orc_td_delta(float q, float r, float m, float lr, float gamma) {
  float target = fmaf(gamma, m, r);
  return lr * (target - q);
}

/* one in-place sample on one table (src/gpu/kernels.cu:7-54, one thread) */
void orc_td_update_one(float* Q, int A, int s, int a, float r, int s2, int done, float lr,
                       float gamma, int mode) {
  float m = orc_next_max(Q + (size_t)s2 * A, A, done, mode);
  Q[(size_t)s * A + a] = orc_td_value(Q[(size_t)s * A + a], r, m, lr, gamma);
}

/* ---- R1: the ordered sum of deltas that hit the same (s,a) ----------------- */
/*
 * Nothing like it exists in the reference (its kernel races on duplicates,
 * src/kernels.cu:114); the order is this build's definition.  Samples (envs)
 * are taken in index order through a fixed three-level tree:
 *
 *   block  = 256 consecutive samples, added left to right from +0.0f
 *   group  = 16 consecutive blocks, block sums added left to right from +0.0f
 *   total  = group sums added left to right from +0.0f
 *   Q[k]   = Q[k] + total[k]   for every k
 *
 * A block or group that holds no sample of a key contributes +0.0f, which
 * changes nothing (a running sum that starts at +0.0f is never -0.0f), so the
 * implementation below only visits the keys a block / group touched.  With at
 * most 256 samples this is plain left-to-right summation.
 */
enum { ORC_BLOCK = 256, ORC_GROUP = 16 };

typedef struct {
  size_t K;
  float *bsum, *gsum, *total;
  int32_t *btouch, *gtouch; /* keys touched in the open block / group */
  uint8_t *bflag, *gflag;
  int nb_touch, ng_touch;
  int in_block, blocks_in_group;
} orc_tree;

static int tree_init(orc_tree* t, size_t K) {
  memset(t, 0, sizeof *t);
  t->K = K;
  t->bsum = (float*)calloc(K, sizeof(float));
  t->gsum = (float*)calloc(K, sizeof(float));
  t->total = (float*)calloc(K, sizeof(float));
  t->btouch = (int32_t*)malloc(ORC_BLOCK * sizeof(int32_t));
  t->gtouch = (int32_t*)malloc((size_t)ORC_BLOCK * ORC_GROUP * sizeof(int32_t));
  t->bflag = (uint8_t*)calloc(K, 1);
  t->gflag = (uint8_t*)calloc(K, 1);
  return (t->bsum && t->gsum && t->total && t->btouch && t->gtouch && t->bflag && t->gflag) ? 0 : -3;
}

static void tree_free(orc_tree* t) {
  free(t->bsum); free(t->gsum); free(t->total);
  free(t->btouch); free(t->gtouch); free(t->bflag); free(t->gflag);
}

static void tree_close_group(orc_tree* t) {
  for (int i = 0; i < t->ng_touch; ++i) {
    int32_t k = t->gtouch[i];
    t->total[k] = t->total[k] + t->gsum[k];
    t->gsum[k] = 0.0f;
    t->gflag[k] = 0;
  }
  t->ng_touch = 0;
  t->blocks_in_group = 0;
}

static void tree_close_block(orc_tree* t) {
  for (int i = 0; i < t->nb_touch; ++i) {
    int32_t k = t->btouch[i];
    t->gsum[k] = t->gsum[k] + t->bsum[k];
    t->bsum[k] = 0.0f;
    t->bflag[k] = 0;
    if (!t->gflag[k]) {
      t->gflag[k] = 1;
      t->gtouch[t->ng_touch++] = k;
    }
  }
  t->nb_touch = 0;
  t->in_block = 0;
  if (++t->blocks_in_group == ORC_GROUP) tree_close_group(t);
}

/* next sample in index order; key < 0 means the sample carries no delta */
static void tree_add(orc_tree* t, int64_t key, float d) {
  if (key >= 0) {
    t->bsum[key] = t->bsum[key] + d;
    if (!t->bflag[key]) {
      t->bflag[key] = 1;
      t->btouch[t->nb_touch++] = (int32_t)key;
    }
  }
  if (++t->in_block == ORC_BLOCK) tree_close_block(t);
}

/* close what is open, apply to Q, and leave the tree empty for the next pass */
static void tree_apply(orc_tree* t, float* Q) {
  if (t->in_block) tree_close_block(t);
  if (t->blocks_in_group) tree_close_group(t);
  for (size_t k = 0; k < t->K; ++k) {
    Q[k] = Q[k] + t->total[k];
    t->total[k] = 0.0f;
  }
}

/* The same sums by the definition, key by key (quadratic: tests only). */
int orc_tree_sum_bruteforce(const int32_t* key, const float* d, int n, int K, float* total) {
  for (int k = 0; k < K; ++k) {
    float tot = 0.0f;
    for (int g0 = 0; g0 < n; g0 += ORC_BLOCK * ORC_GROUP) {
      float gs = 0.0f;
      for (int b0 = g0; b0 < n && b0 < g0 + ORC_BLOCK * ORC_GROUP; b0 += ORC_BLOCK) {
        float bs = 0.0f;
        for (int i = b0; i < n && i < b0 + ORC_BLOCK; ++i)
          if (key[i] == k) bs = bs + d[i];
        gs = gs + bs;
      }
      tot = tot + gs;
    }
    total[k] = tot;
  }
  return 0;
}

/* The tree of the implementation above, exposed for the same test. */
int orc_tree_sum(const int32_t* key, const float* d, int n, int K, float* total) {
  orc_tree t;
  if (tree_init(&t, (size_t)K)) { tree_free(&t); return -3; }
  for (int i = 0; i < n; ++i) tree_add(&t, key[i], d[i]);
  for (int k = 0; k < K; ++k) total[k] = 0.0f;
  tree_apply(&t, total); /* 0 + total */
  tree_free(&t);
  return 0;
}

/* Batch on one table of K = S*A entries (CudaQLearning::update_batch,
 * src/q_learning.cu:108-174): every read sees the table before the call; the
 * deltas are summed per (s,a) through the tree above in sample order and then
 * applied.  Equals the reference up to one rounding when every (s,a) is unique
 * and no written row is another sample's next row.  An action outside [0,A)
 * has no table entry and is skipped. */
int orc_td_update_batch(float* Q, int S, int A, int n, const int32_t* s, const int32_t* a,
                        const float* r, const int32_t* s2, const uint8_t* done, float lr,
                        float gamma, int mode) {
  orc_tree t;
  if (tree_init(&t, (size_t)S * A)) { tree_free(&t); return -3; }
  for (int i = 0; i < n; ++i) {
    if (a[i] < 0 || a[i] >= A) { tree_add(&t, -1, 0.0f); continue; }
    float m = orc_next_max(Q + (size_t)s2[i] * A, A, done[i], mode);
    size_t k = (size_t)s[i] * A + a[i];
    tree_add(&t, (int64_t)k, orc_td_delta(Q[k], r[i], m, lr, gamma));
  }
  tree_apply(&t, Q);
  tree_free(&t);
  return 0;
}

/* ---- epsilon schedule ------------------------------------------------------ */
/* src/train.py:140-141 multiplies a Python float (double) once per update;
 * the table holds those doubles rounded to fp32.  Returns the length. */
int orc_eps_table(const orc_config* c, float* out, int cap) {
  int len = 1;
  if (c->eps_mode == 0) {
    if (cap > 0) out[0] = c->eps0;
    return 1;
  }
  if (c->eps_mode == 1 || c->eps_mode == 2) {
    len = c->eps_span > 0 ? c->eps_span : 1;
    double e = (double)c->eps0;
    for (int i = 0; i < len; ++i) {
      if (i < cap) out[i] = (float)e;
      e *= (double)c->eps_decay;
    }
    return len;
  }
  /* linear: span+1 entries, the last is eps_end */
  int span = c->eps_span > 0 ? c->eps_span : 1;
  len = span + 1;
  for (int i = 0; i < len; ++i) {
    double e = (double)c->eps0 + ((double)c->eps_end - (double)c->eps0) * (double)i / (double)span;
    if (i < cap) out[i] = (float)e;
  }
  return len;
}

static float eps_at(const orc_config* c, const float* tab, int len, uint64_t t, int32_t episode) {
  if (c->eps_mode == 0) return c->eps0;
  uint64_t i = (c->eps_mode == 1) ? t : (uint64_t)(episode < 0 ? 0 : episode);
  if (i >= (uint64_t)len) i = (uint64_t)len - 1;
  return tab[i];
}

/* ---- D1: the driver loop (src/train.py:198-222), batched ------------------ */

static int eps_cap(const orc_config* c) {
  if (c->eps_mode == 1 || c->eps_mode == 2) return c->eps_span > 0 ? c->eps_span : 1;
  if (c->eps_mode == 3) return (c->eps_span > 0 ? c->eps_span : 1) + 1;
  return 1;
}

/* per-env episode statistics (src/train.py:186-226: episode_reward summed step
 * by step, episode_rewards / episode_lengths appended when the episode ends);
 * every pointer indexes one env, or the struct pointer is NULL */
typedef struct {
  float* ret_acc;    /* return of the open episode */
  float* ret_last;   /* return of the last finished episode */
  float* ret_sum;    /* sum over finished episodes */
  int32_t* len_last;
  int32_t* len_sum;
} orc_stats;

/* One env, one step: select (src/train.py:200) -> step (:201) -> update (:205).
 * q is the env's table (or the shared one); with sum != NULL the delta goes
 * into the ordered tree instead of being applied.  Returns s' before any
 * restart, or -1 if the env has used up its episode budget and did nothing. */
static int32_t env_step(const orc_config* c, float eps, float u, int32_t ar, const uint8_t* m_cls,
                        const float* m_cr, float* q, orc_tree* sum, int32_t start, int32_t* s,
                        int32_t* ep_step, int32_t* episode, float* reward, uint8_t* done,
                        uint8_t* action, const orc_stats* st) {
  const int A = c->n_actions;
  if (c->max_episodes > 0 && *episode >= c->max_episodes) {
    if (sum) tree_add(sum, -1, 0.0f);
    return -1;
  }
  int32_t s0 = *s;
  int a = orc_select(q + (size_t)s0 * A, A, eps, u, ar);
  int32_t s2 = s0;
  float r;
  int hit = orc_step_cls(c, m_cls, m_cr, &s2, a, &r);
  int d = hit || (!c->auto_reset && *done);
  float mx = orc_next_max(q + (size_t)s2 * A, A, d, c->max_mode);
  size_t key = (size_t)s0 * A + a;
  if (sum)
    tree_add(sum, (int64_t)key, orc_td_delta(q[key], r, mx, c->lr, c->gamma));
  else
    q[key] = orc_td_value(q[key], r, mx, c->lr, c->gamma);
  *ep_step += 1;
  *reward = r;
  *done = (uint8_t)d;
  *action = (uint8_t)a;
  if (st) *st->ret_acc = *st->ret_acc + r;
  if (c->auto_reset && (d || (c->episode_len > 0 && *ep_step >= c->episode_len))) {
    if (st) {
      *st->ret_last = *st->ret_acc;
      *st->len_last = *ep_step;
      *st->ret_sum = *st->ret_sum + *st->ret_acc;
      *st->len_sum = *st->len_sum + *ep_step;
      *st->ret_acc = 0.0f;
    }
    *s = start;
    *ep_step = 0;
    *episode += 1;
  } else {
    *s = s2;
  }
  return s2;
}

/*
 * n_steps of select -> step -> update for all envs, starting at global step
 * t0.  cls/cr: n_maps maps (1 when map_mode is shared); Q: N tables or one.
 * s, ep_step, episode, reward, done, action: per-env state, in and out.
 * u_sup/a_sup (optional, [n_steps][N]) replace the Philox draws.
 * Trace arrays (optional) are [n_steps][trace_n].
 *
 * Shared table: every env of a step reads the table as it was before the
 * step; the deltas are then summed per (s,a) in env order through the
 * block / group tree defined above, and Q[k] = Q[k] + total[k] for every k.
 */
int orc_run(const orc_config* c, const uint8_t* cls, const float* cr, const int32_t* start,
            float* Q, int32_t* s, int32_t* ep_step, int32_t* episode, float* reward,
            uint8_t* done, uint8_t* action, uint64_t t0, int32_t n_steps, const float* u_sup,
            const int32_t* a_sup, int32_t trace_n, int32_t* tr_s, uint8_t* tr_a, float* tr_r,
            uint8_t* tr_d, float* ret_acc, float* ret_last, float* ret_sum, int32_t* len_last,
            int32_t* len_sum) {
  const int N = c->n_envs, A = c->n_actions;
  const size_t S = (size_t)c->width * c->height;
  const size_t K = S * A;
  const int shared = c->table_mode == 1;
  int cap = eps_cap(c);
  float* tab = (float*)malloc((size_t)cap * sizeof(float));
  orc_tree tree;
  memset(&tree, 0, sizeof tree);
  if (!tab || (shared && tree_init(&tree, K))) {
    free(tab);
    tree_free(&tree);
    return -3;
  }
  orc_tree* sum = shared ? &tree : NULL;
  int len = orc_eps_table(c, tab, cap);

  for (int k = 0; k < n_steps; ++k) {
    uint64_t t = t0 + (uint64_t)k;
    for (int i = 0; i < N; ++i) {
      size_t mo = c->map_mode == 1 ? 0 : (size_t)i * S;
      float u;
      int32_t ar;
      if (u_sup) {
        u = u_sup[(size_t)k * N + i];
        ar = a_sup[(size_t)k * N + i];
      } else {
        orc_explore_draw(c->seed, (uint32_t)i, t, A, &u, &ar);
      }
      float eps = eps_at(c, tab, len, t, episode[i]);
      orc_stats st = {0};
      if (ret_acc) {
        st.ret_acc = ret_acc + i;
        st.ret_last = ret_last + i;
        st.ret_sum = ret_sum + i;
        st.len_last = len_last + i;
        st.len_sum = len_sum + i;
      }
      int32_t s2 = env_step(c, eps, u, ar, cls + mo, cr ? cr + mo : NULL,
                            Q + (shared ? 0 : (size_t)i * K), sum, start[i], &s[i], &ep_step[i],
                            &episode[i], &reward[i], &done[i], &action[i], ret_acc ? &st : NULL);
      if (i < trace_n) {
        size_t o = (size_t)k * trace_n + i;
        if (s2 >= 0) {
          tr_s[o] = s2;
          tr_a[o] = action[i];
          tr_r[o] = reward[i];
          tr_d[o] = done[i];
        } else { /* budget used up: the env stays where it is */
          tr_s[o] = s[i];
          tr_a[o] = 0;
          tr_r[o] = 0.0f;
          tr_d[o] = 0;
        }
      }
    }
    if (shared) tree_apply(sum, Q);
  }
  free(tab);
  tree_free(&tree);
  return 0;
}

/* orc_run for per-env tables restricted to envs [lo, hi), env-major: lets the
 * timing harness spread envs over host threads (envs are independent, and the
 * draws are keyed by the global env index, so the results are orc_run's). */
int orc_run_range(const orc_config* c, int32_t lo, int32_t hi, const uint8_t* cls,
                  const float* cr, const int32_t* start, float* Q, int32_t* s,
                  int32_t* ep_step, int32_t* episode, float* reward, uint8_t* done,
                  uint8_t* action, uint64_t t0, int32_t n_steps) {
  if (c->table_mode == 1) return -1;
  const int A = c->n_actions;
  const size_t S = (size_t)c->width * c->height;
  const size_t K = S * A;
  int cap = eps_cap(c);
  float* tab = (float*)malloc((size_t)cap * sizeof(float));
  if (!tab) return -3;
  int len = orc_eps_table(c, tab, cap);
  for (int i = lo; i < hi; ++i) {
    size_t mo = c->map_mode == 1 ? 0 : (size_t)i * S;
    for (int k = 0; k < n_steps; ++k) {
      uint64_t t = t0 + (uint64_t)k;
      float u;
      int32_t ar;
      orc_explore_draw(c->seed, (uint32_t)i, t, A, &u, &ar);
      float eps = eps_at(c, tab, len, t, episode[i]);
      env_step(c, eps, u, ar, cls + mo, cr ? cr + mo : NULL, Q + (size_t)i * K, NULL, start[i],
               &s[i], &ep_step[i], &episode[i], &reward[i], &done[i], &action[i], NULL);
    }
  }
  free(tab);
  return 0;
}
