/*
 * CPU oracle for the transit-parallel sampling path.  TEST INFRASTRUCTURE ONLY:
 * see nd_oracle.h.  Plain C, compiled with -ffp-contract=off so that every float
 * operation is the single IEEE operation written here.
 */
#include "nd_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* Philox4x32-10                                                              */
/* ------------------------------------------------------------------------- */

void ndo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  /* multipliers and Weyl key increments as published for philox4x32 */
  const uint64_t mul_a = 0xD2511F53u, mul_b = 0xCD9E8D57u;
  const uint32_t weyl_a = 0x9E3779B9u, weyl_b = 0xBB67AE85u;
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int round = 0; round < 10; ++round) {
    uint64_t pa = mul_a * (uint64_t)c0;
    uint64_t pb = mul_b * (uint64_t)c2;
    uint32_t n0 = (uint32_t)(pb >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)pb;
    uint32_t n2 = (uint32_t)(pa >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)pa;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += weyl_a; k1 += weyl_b;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

float ndo_uniform(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw) {
  uint32_t ctr[4] = {(uint32_t)slot, (uint32_t)(slot >> 32), step, draw >> 2};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  ndo_philox4x32_10(ctr, key, out);
  return (float)(out[draw & 3u] >> 8) * 5.9604644775390625e-08f; /* 2^-24 */
}

int32_t ndo_rand_int(float u, int32_t n) {
  /* rand_num_gen.cuh:118-121: ff = u * n (float multiply, n converted to float),
   * id = min((EdgePos_t)ff, n-1) */
  float ff = u * (float)n;
  int32_t id = (int32_t)ff;
  return id < n - 1 ? id : n - 1;
}

float ndo_uniform_grouped(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw) {
  /* steps with stepSize > 1: the first draw of four consecutive slots comes from one block */
  if (draw == 0) return ndo_uniform(seed, slot >> 2, step | 0x80000000u, (uint32_t)(slot & 3u));
  return ndo_uniform(seed, slot, step, draw - 1);
}

/* A cursor over the draws of one (slot, step): what the device RandState is. */
typedef struct {
  uint64_t seed, slot;
  uint32_t step, draw;
  ndo_stats* st;
  int grouped;  /* the step's stepSize is > 1 */
} rng_cursor;

static float next_uniform(rng_cursor* c) {
  float u = c->grouped ? ndo_uniform_grouped(c->seed, c->slot, c->step, c->draw)
                       : ndo_uniform(c->seed, c->slot, c->step, c->draw);
  c->draw++;
  if (c->st) c->st->draws++;
  return u;
}

static int32_t next_int(rng_cursor* c, int32_t n) { return ndo_rand_int(next_uniform(c), n); }

/* ------------------------------------------------------------------------- */
/* Shape algebra                                                              */
/* ------------------------------------------------------------------------- */

int ndo_is_collective(const ndo_app_desc* app) {
  return app->kind == NDO_LAYER_LITERAL || app->kind == NDO_FASTGCN_IMPORTANCE ||
         app->kind == NDO_LADIES_IMPORTANCE;
}

int64_t ndo_step_size_at_step(const ndo_app_desc* app, int step) {
  /* nextdoor.cu:162-186 */
  if (step == -1) return 0;
  if (!ndo_is_collective(app)) {
    int64_t n = app->initial_size;
    for (int i = 0; i <= step; ++i) n *= app->step_size[i];
    return n;
  }
  int64_t n = 0;
  for (int i = 0; i <= step; ++i) n += app->step_size[i];
  return n;
}

int64_t ndo_number_of_transits(const ndo_app_desc* app, int step) {
  /* nextdoor.cu:188-197 */
  if (ndo_is_collective(app)) return app->step_size[step];
  return ndo_step_size_at_step(app, step);
}

int64_t ndo_sub_warp_size_at_step(const ndo_app_desc* app, int step) {
  /* nextdoor.cu:133-160: next power of two >= stepSize(step) */
  if (step == -1) return 0;
  int64_t x = app->step_size[step];
  int64_t w = 1;
  while (w < x) w <<= 1;
  return w;
}

int64_t ndo_final_sample_size(const ndo_app_desc* app) {
  /* nextdoor.cu:1913-1929; individual apps: one entry per output slot, i.e. the product starts
   * at the initial sample size (1 for the reference's walk and k-hop apps) */
  int64_t total = 0, per_step = ndo_is_collective(app) || app->initial_size < 1 ? 1 : app->initial_size;
  for (int k = 0; k < app->steps; ++k) {
    if (ndo_is_collective(app)) per_step = app->step_size[k];
    else per_step *= app->step_size[k];
    total += per_step;
  }
  return total;
}

int ndo_max_bits(int32_t n_vertices) {
  /* nextdoor.cu:1993-1999 with INVALID_VERTEX = n_vertices */
  int bits = 0;
  while (((int64_t)n_vertices >> bits) != 0) bits++;
  return bits;
}

/* ------------------------------------------------------------------------- */
/* Graph accessors                                                            */
/* ------------------------------------------------------------------------- */

static inline int32_t degree_of(const ndo_graph* g, int32_t v) { return g->row_ptr[v + 1] - g->row_ptr[v]; }

/* utils::binarySearch (utils.hpp:30-48) */
static int sorted_contains(const int32_t* a, int32_t x, int32_t n, ndo_stats* st) {
  int32_t l = 0, r = n - 1;
  while (l <= r) {
    int32_t m = l + (r - l) / 2;
    if (st) st->search_probes++;
    if (a[m] == x) return 1;
    if (a[m] < x) l = m + 1; else r = m - 1;
  }
  return 0;
}

int ndo_has_edge(const ndo_graph* g, int32_t src, int32_t dst) {
  return sorted_contains(g->col + g->row_ptr[src], dst, degree_of(g, src), 0);
}

/* ------------------------------------------------------------------------- */
/* next() of the IndividualNeighborhood apps                                  */
/* ------------------------------------------------------------------------- */

static int32_t next_individual(const ndo_graph* g, const ndo_app_desc* app, int step, int32_t transit,
                               int32_t* t_state, rng_cursor* rc) {
  ndo_stats* st = rc->st;
  const int32_t n = degree_of(g, transit);
  const int32_t* edges = g->col + g->row_ptr[transit];
  const float* weights = g->weight + g->row_ptr[transit];
  const float max_w = g->max_weight[transit];
  if (st) st->next_calls++;

  switch (app->kind) {
    case NDO_UNIFORM_WALK: {
      /* example/uniformRandWalk.cu:35-36 (never called with n == 0: nextdoor.cu:257) */
      int32_t x = next_int(rc, n);
      if (st) st->edge_reads++;
      return edges[x];
    }
    case NDO_KHOP: {
      /* khop.cu:18-22 */
      if (n == 0) return -1;
      int32_t x = next_int(rc, n);
      if (st) st->edge_reads++;
      return edges[x];
    }
    case NDO_DEEPWALK:
    case NDO_PPR: {
      if (n == 0) return -1;
      if (app->kind == NDO_PPR) {
        /* randomWalks.cu:105-109 */
        float stop = next_uniform(rc);
        if (stop < 0.01f) return -1;
      }
      if (n == 1) { if (st) st->edge_reads++; return edges[0]; }
      /* randomWalks.cu:81-88: rejection against the vertex's max edge weight */
      int32_t x = next_int(rc, n);
      float y = next_uniform(rc) * max_w;
      if (st) st->weight_reads++;
      while (y > weights[x]) {
        x = next_int(rc, n);
        y = next_uniform(rc) * max_w;
        if (st) st->weight_reads++;
      }
      if (st) st->edge_reads++;
      return edges[x];
    }
    case NDO_NODE2VEC: {
      /* randomWalks.cu:141-172, literally: the return-edge test compares the edge
       * INDEX x with the vertex id t (randomWalks.cu:159). */
      if (n == 0) return -1;
      if (n == 1 || step == 0) { *t_state = transit; if (st) st->edge_reads++; return edges[0]; }
      const float p = app->p, q = app->q;
      float envelope = p > 1.0f / q ? p : 1.0f / q;
      if (envelope < 1.0f) envelope = 1.0f;
      for (;;) {
        int32_t x = next_int(rc, n);
        int32_t v = edges[x];
        if (st) st->edge_reads++;
        float y = next_uniform(rc) * envelope;
        int32_t t = *t_state;
        float h;
        if (x == t) h = p;
        else if (sorted_contains(g->col + g->row_ptr[t], v, degree_of(g, t), st)) h = 1.0f / q;
        else h = 1.0f;
        if (y < h) { *t_state = transit; return v; }
      }
    }
    case NDO_WEIGHTED_NODE2VEC: {
      /* Own definition (the reference has no weighted node2vec): second-order bias h
       * as above but with the return test on the VERTEX (v == t), multiplied by the
       * edge weight, rejected against max_weight * max(p, 1/q, 1).  Step 0 has no
       * previous vertex: h = 1, i.e. a DeepWalk step. */
      if (n == 0) return -1;
      if (n == 1) { *t_state = transit; if (st) st->edge_reads++; return edges[0]; }
      const float p = app->p, q = app->q;
      float hmax = p > 1.0f / q ? p : 1.0f / q;
      if (hmax < 1.0f) hmax = 1.0f;
      float hmin = p < 1.0f / q ? p : 1.0f / q;
      if (hmin > 1.0f) hmin = 1.0f;
      const float envelope = max_w * hmax;
      for (;;) {
        int32_t x = next_int(rc, n);
        int32_t v = edges[x];
        float wx = weights[x];
        if (st) { st->edge_reads++; st->weight_reads++; }
        float y = next_uniform(rc) * envelope;
        float h;
        if (st && step > 0 && !(y < hmin * wx) && y < hmax * wx) st->band_tests++;  /* statistics only */
        if (step == 0) h = 1.0f;
        else {
          int32_t t = *t_state;
          if (v == t) h = p;
          else if (sorted_contains(g->col + g->row_ptr[t], v, degree_of(g, t), st)) h = 1.0f / q;
          else h = 1.0f;
        }
        if (y < h * wx) { *t_state = transit; return v; }
      }
    }
    default:
      return -1;
  }
}

int ndo_sample_individual(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                          int64_t n_samples, int64_t first_sample,
                          const int32_t* initial, int32_t* final_samples,
                          int32_t* state_t, ndo_stats* stats, int n_threads) {
  if (ndo_is_collective(app) || app->steps <= 0 || app->steps > NDO_MAX_STEPS) return -1;
  const int32_t invalid = g->n_vertices;
  const int64_t F = ndo_final_sample_size(app);
  const int init = app->initial_size;
  if (stats) memset(stats, 0, sizeof(*stats));
  if (n_threads < 1) n_threads = 1;

  ndo_stats* per_thread = (ndo_stats*)calloc((size_t)n_threads, sizeof(ndo_stats));
  if (!per_thread) return -2;

#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 256) num_threads(n_threads)
#endif
  for (int64_t s = 0; s < n_samples; ++s) {
    int tid = 0;
#ifdef _OPENMP
    tid = omp_get_thread_num();
#endif
    ndo_stats* st = stats ? &per_thread[tid] : 0;
    int32_t* out = final_samples + s * F;
    int32_t t_state = -1;
    const int32_t* prev = initial + s * init;  /* transits of step k */
    int64_t T = init;                          /* numberOfTransits of step k-1 / transits per sample */
    int64_t seg_base = 0;
    for (int k = 0; k < app->steps; ++k) {
      const int m = app->step_size[k];
      int32_t* seg = out + seg_base;
      for (int64_t j = 0; j < T; ++j) {
        const int32_t transit = prev[j];
        for (int nbr = 0; nbr < m; ++nbr) {
          int32_t neighbor = invalid;
          /* nextdoor.cu:250-262: next() only runs for a valid transit with edges */
          if (transit != invalid && transit != -1 && degree_of(g, transit) != 0) {
            rng_cursor rc;
            rc.seed = seed;
            rc.slot = (uint64_t)(((first_sample + s) * T + j) * m + nbr);
            rc.step = (uint32_t)k;
            rc.draw = 0;
            rc.st = st;
            rc.grouped = m > 1;
            int32_t r = next_individual(g, app, k, transit, &t_state, &rc);
            neighbor = (r == -1) ? invalid : r;  /* nextdoor.cu:288 */
          }
          seg[j * m + nbr] = neighbor;
          if (st && neighbor != invalid) st->valid_outputs++;
        }
      }
      prev = seg;
      seg_base += T * m;
      T *= m;
    }
    if (state_t) state_t[s] = t_state;
  }

  if (stats) {
    for (int i = 0; i < n_threads; ++i) {
      stats->next_calls += per_thread[i].next_calls;
      stats->draws += per_thread[i].draws;
      stats->search_probes += per_thread[i].search_probes;
      stats->valid_outputs += per_thread[i].valid_outputs;
      stats->edge_reads += per_thread[i].edge_reads;
      stats->weight_reads += per_thread[i].weight_reads;
      stats->band_tests += per_thread[i].band_tests;
    }
  }
  free(per_thread);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Multi-dimensional random walk                                              */
/* ------------------------------------------------------------------------- */

/* start vertex of walker root_index of a sample: a fixed Philox stream ("MRWR") */
int32_t ndo_multirw_root(int64_t sample, int root_index, int32_t n_vertices) {
  const float u = ndo_uniform(0x4D525752ull, (uint64_t)sample, 0x524F4F54u, (uint32_t)root_index);
  return ndo_rand_int(u, n_vertices);
}

int ndo_sample_multirw(const ndo_graph* g, uint64_t seed, int64_t n_samples, int64_t first_sample, int n_roots,
                       int steps, int32_t* roots, int32_t* last_root_idx, int32_t* final_samples,
                       int32_t* transits_out) {
  if (steps <= 0 || steps > NDO_MAX_STEPS || n_roots <= 0) return -1;
  const int32_t invalid = g->n_vertices;
  for (int64_t s = 0; s < n_samples; ++s) {
    int32_t* walkers = roots + s * n_roots;
    int32_t last_idx = 0;
    int32_t transit = walkers[0];  /* multiRW.cu:68-73: the initial sample is walker 0 */
    for (int k = 0; k < steps; ++k) {
      if (transits_out) transits_out[s * steps + k] = transit;
      rng_cursor rc;
      rc.seed = seed;
      rc.slot = (uint64_t)(first_sample + s);
      rc.step = (uint32_t)k;
      rc.draw = 0;
      rc.st = 0;
      rc.grouped = 0;
      int32_t neighbor = invalid;
      if (transit != invalid && degree_of(g, transit) != 0) {
        const int32_t n = degree_of(g, transit);
        const int32_t* edges = g->col + g->row_ptr[transit];
        int32_t v = n == 1 ? edges[0] : edges[next_int(&rc, n)];  /* multiRW.cu:31-43 */
        if (k > 0) walkers[last_idx] = v;                          /* multiRW.cu:34-36, 45-47 */
        neighbor = v;
      }
      final_samples[s * steps + k] = neighbor;
      if (k != steps - 1) {                                        /* nextdoor.cu:282-286 */
        last_idx = next_int(&rc, n_roots);                         /* multiRW.cu:88-91 */
        transit = walkers[last_idx];
      }
    }
    if (last_root_idx) last_root_idx[s] = last_idx;
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Explicit transits with several transits per sample                         */
/* ------------------------------------------------------------------------- */

int ndo_sample_anchor_hop(const ndo_graph* g, uint64_t seed, int64_t n_samples, int64_t first_sample,
                          int n_anchors, const int32_t* anchors, int steps, const int* step_size,
                          int32_t* final_samples, int32_t* transits_out) {
  if (steps <= 0 || steps > NDO_MAX_STEPS || n_anchors <= 0) return -1;
  const int32_t invalid = g->n_vertices;
  int64_t F = 0, widest = n_anchors, per_step = n_anchors;
  for (int k = 0; k < steps; ++k) {
    per_step *= step_size[k];
    F += per_step;
    if (per_step > widest) widest = per_step;
  }
  int32_t* map_a = (int32_t*)malloc(sizeof(int32_t) * (size_t)widest);
  int32_t* map_b = (int32_t*)malloc(sizeof(int32_t) * (size_t)widest);
  if (!map_a || !map_b) { free(map_a); free(map_b); return -2; }
  for (int64_t s = 0; s < n_samples; ++s) {
    const int32_t* mine = anchors + s * n_anchors;
    int32_t* out = final_samples + s * F;
    int32_t* prev = map_a;
    int32_t* next = map_b;
    for (int i = 0; i < n_anchors; ++i) prev[i] = mine[i];  /* the initial sample: the anchors */
    int64_t T = n_anchors, seg_base = 0;
    for (int k = 0; k < steps; ++k) {
      const int m = step_size[k];
      for (int64_t j = 0; j < T; ++j) {
        const int32_t transit = prev[j];
        if (transits_out) transits_out[s * F + seg_base + j * m] = transit;  /* the transit its outputs were drawn from */
        for (int nbr = 0; nbr < m; ++nbr) {
          int32_t neighbor = invalid, chosen = invalid;
          if (transit != invalid && transit != -1) {  /* a pair without a transit is dead, and so is what follows it */
            rng_cursor rc;
            rc.seed = seed;
            rc.slot = (uint64_t)(((first_sample + s) * T + j) * m + nbr);
            rc.step = (uint32_t)k;
            rc.draw = 0;
            rc.st = 0;
            rc.grouped = m > 1;
            const int32_t n = degree_of(g, transit);
            if (n != 0) neighbor = g->col[g->row_ptr[transit] + next_int(&rc, n)];  /* nextdoor.cu:250-262, khop.cu:18-22 */
            if (k != steps - 1) {
              /* nextdoor.cu:279-289: stepTransits(k + 1) with the random state next() used and
               * the index (thread number) % (transits per sample of this step) */
              const int64_t index = (j * m + nbr) % T;
              const int32_t x = next_int(&rc, n_anchors + 1);
              if (x != n_anchors) chosen = mine[(index + x) % n_anchors];
            }
          }
          out[seg_base + j * m + nbr] = neighbor;
          next[j * m + nbr] = chosen;
        }
      }
      int32_t* swap = prev; prev = next; next = swap;
      seg_base += T * m;
      T *= m;
    }
  }
  free(map_a);
  free(map_b);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Inversion / RLE / scan / binning                                           */
/* ------------------------------------------------------------------------- */

void ndo_sort_pairs(const int32_t* keys_in, const int32_t* vals_in, int64_t n,
                    int32_t* keys_out, int32_t* vals_out) {
  /* stable counting-free merge sort on indices: simple and obviously stable */
  if (n <= 0) return;
  int64_t* idx = (int64_t*)malloc(sizeof(int64_t) * (size_t)n);
  int64_t* tmp = (int64_t*)malloc(sizeof(int64_t) * (size_t)n);
  for (int64_t i = 0; i < n; ++i) idx[i] = i;
  for (int64_t width = 1; width < n; width *= 2) {
    for (int64_t lo = 0; lo < n; lo += 2 * width) {
      int64_t mid = lo + width < n ? lo + width : n;
      int64_t hi = lo + 2 * width < n ? lo + 2 * width : n;
      int64_t a = lo, b = mid, o = lo;
      while (a < mid && b < hi) {
        /* take from the left run on ties: stability */
        if ((uint32_t)keys_in[idx[b]] < (uint32_t)keys_in[idx[a]]) tmp[o++] = idx[b++];
        else tmp[o++] = idx[a++];
      }
      while (a < mid) tmp[o++] = idx[a++];
      while (b < hi) tmp[o++] = idx[b++];
    }
    int64_t* sw = idx; idx = tmp; tmp = sw;
  }
  for (int64_t i = 0; i < n; ++i) {
    keys_out[i] = keys_in[idx[i]];
    vals_out[i] = vals_in[idx[i]];
  }
  free(idx);
  free(tmp);
}

int64_t ndo_unique_transits(const int32_t* sorted_keys, int64_t n, int32_t invalid,
                            int32_t* uniq, int32_t* counts, int32_t* offsets,
                            int64_t* n_valid) {
  /* invalidVertexStartPos (nextdoor.cu:1804-1836) + RunLengthEncode (2535-2545)
   * + ExclusiveSum (2560-2567) */
  int64_t valid = 0;
  while (valid < n && sorted_keys[valid] != invalid) valid++;
  if (n_valid) *n_valid = valid;
  int64_t runs = 0;
  for (int64_t i = 0; i < valid;) {
    int64_t j = i;
    while (j < valid && sorted_keys[j] == sorted_keys[i]) j++;
    uniq[runs] = sorted_keys[i];
    counts[runs] = (int32_t)(j - i);
    offsets[runs] = (int32_t)i;
    runs++;
    i = j;
  }
  return runs;
}

int ndo_kernel_class(int64_t count, int64_t sub_warp_size) {
  int64_t work = count * sub_warp_size;
  if (work >= 256) return 1;
  if (work >= 32) return 2;
  if (work >= 8) return 3;
  return 4;
}

/* ------------------------------------------------------------------------- */
/* Distinct                                                                   */
/* ------------------------------------------------------------------------- */

static int cmp_i32(const void* a, const void* b) {
  int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
  return (x > y) - (x < y);
}

void ndo_distinct(const ndo_app_desc* app, int64_t n_samples, int32_t invalid,
                  int32_t* final_samples, int32_t* counts) {
  const int64_t F = ndo_final_sample_size(app);
  for (int64_t s = 0; s < n_samples; ++s) {
    int64_t base = 0;
    for (int k = 0; k < app->steps; ++k) {
      int64_t len = ndo_step_size_at_step(app, k);
      int32_t* seg = final_samples + s * F + base;
      /* invalid == n_vertices is larger than every vertex id, so it sorts last */
      qsort(seg, (size_t)len, sizeof(int32_t), cmp_i32);
      int64_t kept = 0;
      for (int64_t i = 0; i < len; ++i) {
        if (seg[i] == invalid) break;
        if (kept == 0 || seg[kept - 1] != seg[i]) seg[kept++] = seg[i];
      }
      for (int64_t i = kept; i < len; ++i) seg[i] = invalid;
      if (counts) counts[s * app->steps + k] = (int32_t)kept;
      base += len;
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Validators                                                                 */
/* ------------------------------------------------------------------------- */

/* numNeighborsSampledAtStep (check_results.cu:4-29), as written */
static int64_t neighbors_sampled_at_step(const ndo_app_desc* app, int step) {
  if (step < 0) return 0;
  int64_t n = app->step_size[0];
  for (int i = 1; i <= step; ++i) {
    if (app->step_size[i] == 1) n += app->step_size[i];
    else n += n * app->step_size[i];
  }
  return n;
}

int ndo_check_sampled_vertices(const ndo_graph* g, const ndo_app_desc* app,
                               int64_t n_samples, const int32_t* initial,
                               const int32_t* final_samples, int32_t invalid, int n_threads) {
  const int64_t F = ndo_final_sample_size(app);
  const int max_steps = 4; /* check_results.cu:173 */
  const int steps = app->steps < max_steps ? app->steps : max_steps;
  int ok = 1;
  if (n_threads < 1) n_threads = 1;
  for (int step = 0; step < steps; ++step) {
    int bad = 0;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads) reduction(| : bad)
#endif
    for (int64_t s = 0; s < n_samples; ++s) {
      const int32_t* fs = final_samples + s * F;
      if (step == 0) {
        /* check_results.cu:185-232 (fixed step sizes only) */
        const int32_t root = initial[s]; /* literal: initialSamples[sampleId] */
        int64_t valid = 0;
        for (int64_t v = 0; v < app->step_size[0]; ++v) {
          int32_t x = fs[v];
          if (x != invalid) {
            valid++;
            if (!ndo_has_edge(g, root, x)) bad |= 1;
          }
        }
        if (valid == 0 && degree_of(g, root) > 0) bad |= 1;
      } else {
        /* check_results.cu:234-291 */
        const int64_t prev_lo = neighbors_sampled_at_step(app, step - 2);
        const int64_t prev_hi = neighbors_sampled_at_step(app, step - 1);
        const int64_t cur_hi = (step == app->steps - 1) ? F : neighbors_sampled_at_step(app, step);
        int64_t prev_edges = 0, valid = 0;
        for (int64_t v = prev_lo; v < prev_hi; ++v)
          if (fs[v] != invalid) prev_edges += degree_of(g, fs[v]);
        for (int64_t v = prev_hi; v < cur_hi; ++v) {
          int32_t x = fs[v];
          if (x == invalid) continue;
          valid++;
          int found = 0;
          for (int64_t v1 = prev_lo; v1 < prev_hi && !found; ++v1)
            if (fs[v1] != invalid && ndo_has_edge(g, fs[v1], x)) found = 1;
          if (!found) bad |= 1;
        }
        if (valid == 0 && prev_edges > 0) bad |= 1;
      }
    }
    if (bad) { ok = 0; break; }
  }
  return ok;
}

int ndo_check_exact_transits(const ndo_graph* g, const ndo_app_desc* app,
                             int64_t n_samples, const int32_t* initial,
                             const int32_t* final_samples, int32_t invalid) {
  const int64_t F = ndo_final_sample_size(app);
  for (int64_t s = 0; s < n_samples; ++s) {
    const int32_t* prev = initial + s * app->initial_size;
    int64_t T = app->initial_size, base = 0;
    for (int k = 0; k < app->steps; ++k) {
      const int m = app->step_size[k];
      const int32_t* seg = final_samples + s * F + base;
      for (int64_t j = 0; j < T; ++j)
        for (int nbr = 0; nbr < m; ++nbr) {
          int32_t x = seg[j * m + nbr];
          if (x < 0 || x > invalid) return 0;
          if (x == invalid) continue;
          if (prev[j] == invalid || !ndo_has_edge(g, prev[j], x)) return 0;
        }
      prev = seg;
      base += T * m;
      T *= m;
    }
  }
  return 1;
}

/* ------------------------------------------------------------------------- */
/* CollectiveNeighborhood sampling                                            */
/* ------------------------------------------------------------------------- */

int64_t ndo_collective_neighborhood(const ndo_graph* g, const int32_t* transits, int n_transits,
                                    int32_t invalid, int32_t* cols, float* weights, int32_t* row_offsets) {
  int64_t size = 0;
  for (int i = 0; i < n_transits; ++i) {
    if (row_offsets) row_offsets[i] = (int32_t)size;
    const int32_t t = transits[i];
    if (t == invalid || t == -1) continue;
    const int32_t b = g->row_ptr[t], e = g->row_ptr[t + 1];
    for (int32_t x = b; x < e; ++x) {
      if (cols) cols[size] = g->col[x];
      if (weights) weights[size] = g->weight[x];
      size++;
    }
  }
  return size;
}

/* transits of sample-row `row` at step k, and how many there are */
static const int32_t* layer_transits(const ndo_app_desc* app, int k, const int32_t* initial_of_sample,
                                     const int32_t* row, int* count) {
  if (k == 0) { *count = app->initial_size; return initial_of_sample; }
  *count = app->step_size[k - 1];
  return row + ndo_step_size_at_step(app, k - 2);
}

int ndo_sample_layer_literal(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                             int64_t n_samples, int64_t first_sample, const int32_t* initial,
                             int32_t* final_samples, int32_t* rows, int32_t* cols, int n_threads) {
  if (!ndo_is_collective(app)) return -1;
  const int32_t invalid = g->n_vertices;
  const int64_t F = ndo_final_sample_size(app);
  const int B = app->initial_size; /* VERTICES_PER_SAMPLE; the reference's apps use it for every layer */
  if (n_threads < 1) n_threads = 1;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4) num_threads(n_threads)
#endif
  for (int64_t s = 0; s < n_samples; ++s) {
    int32_t* row = final_samples + s * F;
    for (int k = 0; k < app->steps; ++k) {
      const int m = app->step_size[k];
      int n_tr;
      const int32_t* transits = layer_transits(app, k, initial + s * app->initial_size, row, &n_tr);
      int32_t* out = row + ndo_step_size_at_step(app, k - 1);
      for (int nbr = 0; nbr < m; ++nbr) {
        int32_t neighbor = invalid;
        /* nextdoor.cu:1421: only the first transit is looked at */
        if (transits[0] != invalid && transits[0] != -1) {
          rng_cursor rc;
          rc.seed = seed; rc.slot = (uint64_t)((first_sample + s) * m + nbr); rc.step = (uint32_t)k;
          rc.draw = 0; rc.st = 0; rc.grouped = 0;
          const int32_t id = next_int(&rc, g->n_vertices);
          for (int i = 0; i < B; ++i) {
            const int has = ndo_has_edge(g, transits[i], id);
            const int64_t len = (int64_t)i * B + nbr;
            const int64_t at = (s * app->steps + k) * (int64_t)B * B + len;
            rows[at] = has ? i : -1;
            cols[at] = has ? nbr : -1;
          }
          neighbor = id;
        }
        out[nbr] = neighbor;
      }
    }
  }
  return 0;
}

int ndo_check_adjacency_matrix(const ndo_graph* g, const ndo_app_desc* app, int64_t n_samples,
                               const int32_t* initial, const int32_t* final_samples,
                               const int32_t* rows, const int32_t* cols, int32_t invalid) {
  const int64_t F = ndo_final_sample_size(app);
  const int B = app->initial_size;
  const int max_steps = app->steps < 4 ? app->steps : 4; /* check_results.cu:57 */
  int64_t sampled_before = 0; /* numNeighborsToSampleAtStep */
  for (int step = 0; step < max_steps; ++step) {
    const int64_t cur = step == 0 ? 0 : sampled_before + app->step_size[step]; /* check_results.cu:66 */
    for (int64_t s = 0; s < n_samples; ++s) {
      const int32_t* fs = final_samples + s * F;
      const int32_t* r = rows + (s * app->steps + step) * (int64_t)B * B;
      const int32_t* c = cols + (s * app->steps + step) * (int64_t)B * B;
      const int64_t len = (int64_t)B * B; /* adjacencyMatrixLen stays 0 -> B*B (check_results.cu:76-79) */
      /* 1: every recorded pair is an edge of the graph */
      for (int64_t v = 0; v < len; ++v) {
        if (c[v] == -1 && r[v] == -1) continue;
        const int32_t to = fs[cur + c[v]];
        const int32_t from = step == 0 ? initial[s * app->initial_size + r[v]] : fs[sampled_before + r[v]];
        if (to != invalid && !ndo_has_edge(g, from, to)) return 0;
      }
      /* 2: every edge between the two layers is recorded */
      const int prev_n = step == 0 ? app->initial_size : app->step_size[step - 1];
      for (int v = 0; v < app->step_size[step]; ++v) {
        const int32_t to = fs[cur + v];
        for (int pi = 0; pi < prev_n; ++pi) {
          const int32_t from = step == 0 ? initial[s * app->initial_size + pi] : fs[sampled_before + pi];
          if (to == invalid || !ndo_has_edge(g, from, to)) continue;
          int found = 0;
          for (int64_t e = 0; e < len && !found; ++e) {
            if (c[e] == -1 && r[e] == -1) continue;
            const int32_t v1 = step == 0 ? initial[s * app->initial_size + r[e]] : fs[sampled_before + r[e]];
            const int32_t v2 = fs[cur + c[e]];
            if (v1 == from && v2 == to) found = 1;
          }
          if (!found) return 0;
        }
      }
    }
    if (step >= 1) sampled_before += app->step_size[step];
  }
  return 1;
}

int ndo_sample_fastgcn_importance(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                                  int64_t n_samples, int64_t first_sample, const int32_t* initial,
                                  int32_t* final_samples, ndo_stats* stats, int n_threads) {
  if (!ndo_is_collective(app)) return -1;
  const int32_t invalid = g->n_vertices;
  const int64_t F = ndo_final_sample_size(app);
  if (stats) memset(stats, 0, sizeof(*stats));
  if (n_threads < 1) n_threads = 1;
  int64_t total_edges = 0, total_distinct = 0, total_valid = 0;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4) num_threads(n_threads) reduction(+ : total_edges, total_distinct, total_valid)
#endif
  for (int64_t s = 0; s < n_samples; ++s) {
    int32_t* row = final_samples + s * F;
    for (int k = 0; k < app->steps; ++k) {
      const int m = app->step_size[k];
      int n_tr;
      const int32_t* transits = layer_transits(app, k, initial + s * app->initial_size, row, &n_tr);
      int32_t* out = row + ndo_step_size_at_step(app, k - 1);
      const int64_t size = ndo_collective_neighborhood(g, transits, n_tr, invalid, 0, 0, 0);
      int32_t* nb = (int32_t*)malloc(sizeof(int32_t) * (size_t)(size > 0 ? size : 1));
      ndo_collective_neighborhood(g, transits, n_tr, invalid, nb, 0, 0);
      qsort(nb, (size_t)size, sizeof(int32_t), cmp_i32);
      int64_t distinct = 0;
      for (int64_t i = 0; i < size; ++i)
        if (distinct == 0 || nb[distinct - 1] != nb[i]) nb[distinct++] = nb[i];
      uint64_t* prefix = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)(distinct > 0 ? distinct : 1));
      uint64_t total = 0;
      for (int64_t i = 0; i < distinct; ++i) {
        const uint64_t d = (uint64_t)degree_of(g, nb[i]);
        total += d * d;
        prefix[i] = total;
      }
      for (int nbr = 0; nbr < m; ++nbr) {
        int32_t pick = invalid;
        if (distinct > 0 && total > 0) {
          uint32_t ctr[4] = {0, 0, (uint32_t)k, 0}, key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)}, w[4];
          const uint64_t slot = (uint64_t)((first_sample + s) * m + nbr);
          ctr[0] = (uint32_t)slot; ctr[1] = (uint32_t)(slot >> 32);
          ndo_philox4x32_10(ctr, key, w);
          const uint64_t r = w[0] >> 8;
          const uint64_t target = (uint64_t)(((unsigned __int128)r * total) >> 24);
          int64_t lo = 0, hi = distinct; /* first i with prefix[i] > target */
          while (lo < hi) {
            const int64_t mid = lo + (hi - lo) / 2;
            if (prefix[mid] > target) hi = mid; else lo = mid + 1;
          }
          pick = nb[lo];
          total_valid++;
        }
        out[nbr] = pick;
      }
      total_edges += size;
      total_distinct += distinct;
      free(prefix);
      free(nb);
    }
  }
  if (stats) {
    stats->edge_reads = total_edges;      /* sum of collective-neighbourhood sizes */
    stats->search_probes = total_distinct; /* sum of distinct counts */
    stats->valid_outputs = total_valid;
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* LADIES importance sampling                                                 */
/* ------------------------------------------------------------------------- */

float ndo_det_log2(float x) {
  uint32_t bits;
  memcpy(&bits, &x, sizeof(bits));
  int e = (int)(bits >> 23) - 127;
  uint32_t mbits = (bits & 0x7FFFFFu) | 0x3F800000u;
  float m;
  memcpy(&m, &mbits, sizeof(m));
  if (m > 1.41421354f) { m = m * 0.5f; e += 1; }
  const float z = (m - 1.0f) / (m + 1.0f);
  const float z2 = z * z;
  float poly = z2 * 0.142857149f; /* 1 + z^2/3 + z^4/5 + z^6/7 by Horner */
  poly = poly + 0.2f;
  poly = poly * z2;
  poly = poly + 0.333333343f;
  poly = poly * z2;
  poly = poly + 1.0f;
  float ln_m = z * poly;
  ln_m = ln_m * 2.0f;
  return (float)e + ln_m * 1.44269502f;
}

static uint32_t descending_key_bits(float key) {
  /* monotone float -> uint32, then inverted so that an ascending sort gives descending keys */
  uint32_t b;
  memcpy(&b, &key, sizeof(b));
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return ~b;
}

/* (weight * (1 / rowsum))^2 as a 2^53 fixed-point integer (exact scaling, truncation) */
static uint64_t term_fixed(float term) {
  if (!(term > 0.0f)) return 0;
  if (term >= 1.0f) return (uint64_t)1 << 53;
  return (uint64_t)(term * 9007199254740992.0f);
}

typedef struct { int32_t vertex; int64_t pos; } occ_t;
static int cmp_occ(const void* a, const void* b) {
  const occ_t* x = (const occ_t*)a; const occ_t* y = (const occ_t*)b;
  if (x->vertex != y->vertex) return (x->vertex > y->vertex) - (x->vertex < y->vertex);
  return (x->pos > y->pos) - (x->pos < y->pos);
}
typedef struct { uint32_t key; int32_t vertex; } ranked_t;
static int cmp_ranked(const void* a, const void* b) {
  const ranked_t* x = (const ranked_t*)a; const ranked_t* y = (const ranked_t*)b;
  if (x->key != y->key) return (x->key > y->key) - (x->key < y->key);
  return (x->vertex > y->vertex) - (x->vertex < y->vertex);
}

int ndo_sample_ladies_importance(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                                 int64_t n_samples, int64_t first_sample, const int32_t* initial,
                                 int32_t* final_samples, ndo_stats* stats, int n_threads) {
  if (!ndo_is_collective(app)) return -1;
  const int32_t invalid = g->n_vertices;
  const int64_t F = ndo_final_sample_size(app);
  if (stats) memset(stats, 0, sizeof(*stats));
  if (n_threads < 1) n_threads = 1;
  /* row sums in edge order */
  float* rowsum = (float*)malloc(sizeof(float) * (size_t)g->n_vertices);
  for (int32_t v = 0; v < g->n_vertices; ++v) {
    float acc = 0.0f;
    for (int32_t x = g->row_ptr[v]; x < g->row_ptr[v + 1]; ++x) acc = acc + g->weight[x];
    rowsum[v] = acc;
  }
  int64_t total_edges = 0, total_distinct = 0, total_valid = 0;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads) reduction(+ : total_edges, total_distinct, total_valid)
#endif
  for (int64_t s = 0; s < n_samples; ++s) {
    int32_t* row = final_samples + s * F;
    for (int k = 0; k < app->steps; ++k) {
      const int m = app->step_size[k];
      int n_tr;
      const int32_t* transits = layer_transits(app, k, initial + s * app->initial_size, row, &n_tr);
      int32_t* out = row + ndo_step_size_at_step(app, k - 1);
      const int64_t size = ndo_collective_neighborhood(g, transits, n_tr, invalid, 0, 0, 0);
      occ_t* occ = (occ_t*)malloc(sizeof(occ_t) * (size_t)(size > 0 ? size : 1));
      float* term = (float*)malloc(sizeof(float) * (size_t)(size > 0 ? size : 1));
      int64_t at = 0;
      for (int i = 0; i < n_tr; ++i) {
        const int32_t u = transits[i];
        if (u == invalid || u == -1) continue;
        for (int32_t x = g->row_ptr[u]; x < g->row_ptr[u + 1]; ++x) {
          const float p = g->weight[x] * (1.0f / rowsum[u]);
          term[at] = p * p;
          occ[at].vertex = g->col[x];
          occ[at].pos = at;
          at++;
        }
      }
      qsort(occ, (size_t)size, sizeof(occ_t), cmp_occ);
      ranked_t* ranked = (ranked_t*)malloc(sizeof(ranked_t) * (size_t)(size > 0 ? size : 1));
      int64_t distinct = 0;
      for (int64_t i = 0; i < size;) {
        int64_t j = i;
        uint64_t imp_fixed = 0;
        while (j < size && occ[j].vertex == occ[i].vertex) { imp_fixed += term_fixed(term[occ[j].pos]); j++; }
        const float imp = (float)imp_fixed;
        const int32_t v = occ[i].vertex;
        uint32_t ctr[4], key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)}, w[4];
        /* four vertices share a Philox block: pair index P = sample * (|V| rounded up to a
         * multiple of 4) + v, block P >> 2, word P & 3 */
        const uint64_t padded_vertices = ((uint64_t)g->n_vertices + 3u) & ~(uint64_t)3;
        const uint64_t pair = (uint64_t)(first_sample + s) * padded_vertices + (uint64_t)v;
        const uint64_t block = pair >> 2;
        ctr[0] = (uint32_t)block; ctr[1] = (uint32_t)(block >> 32); ctr[2] = (uint32_t)k; ctr[3] = 0;
        ndo_philox4x32_10(ctr, key, w);
        const float u01 = ((float)(w[pair & 3u] >> 8) + 0.5f) * 5.9604644775390625e-08f;
        float keyf;
        if (imp > 0.0f) keyf = ndo_det_log2(u01) / imp;
        else keyf = -__builtin_inff();
        ranked[distinct].key = descending_key_bits(keyf);
        ranked[distinct].vertex = v;
        distinct++;
        i = j;
      }
      qsort(ranked, (size_t)distinct, sizeof(ranked_t), cmp_ranked);
      for (int nbr = 0; nbr < m; ++nbr) {
        out[nbr] = nbr < distinct ? ranked[nbr].vertex : invalid;
        if (nbr < distinct) total_valid++;
      }
      total_edges += size;
      total_distinct += distinct;
      free(ranked); free(term); free(occ);
    }
  }
  free(rowsum);
  if (stats) {
    stats->edge_reads = total_edges;
    stats->search_probes = total_distinct;
    stats->valid_outputs = total_valid;
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Edge-list apps: MVS and ClusterGCN                                         */
/* ------------------------------------------------------------------------- */

int64_t ndo_subgraph_num_samples(const ndo_graph* g, int vertices_per_sample, int64_t cap) {
  if (g->n_edges > 100000000) return 800000;
  const int64_t wanted = ((int64_t)g->n_vertices * 8 + vertices_per_sample - 1) / vertices_per_sample;
  return wanted < cap ? wanted : cap;
}

void ndo_mvs_vertices(const ndo_graph* g, int64_t n_samples, int batch, int32_t* vertices) {
  for (int64_t s = 0; s < n_samples; ++s)
    for (int i = 0; i < batch; ++i) vertices[s * batch + i] = (int32_t)((s * batch + i) % g->n_vertices);
}

void ndo_clustergcn_vertices(const ndo_graph* g, int64_t n_samples, int cluster_size, int clusters_per_sample,
                             int32_t* vertices) {
  const int64_t n_clusters = g->n_vertices / cluster_size;
  for (int64_t s = 0; s < n_samples; ++s) {
    int32_t* mine = vertices + s * cluster_size * clusters_per_sample;
    for (int i = 0; i < clusters_per_sample; ++i) {
      const int64_t c = (s * clusters_per_sample + i) % n_clusters;
      for (int v = 0; v < cluster_size; ++v) *mine++ = (int32_t)(c * cluster_size + v);
    }
  }
}

int64_t ndo_sample_mvs(const ndo_graph* g, int64_t n_samples, int batch, const int32_t* vertices,
                       uint32_t* list_start, int32_t* rows, int32_t* cols) {
  const int64_t lanes = (int64_t)batch * batch;  /* lane l = j * batch + nbr */
  int64_t at = 0;
  for (int64_t s = 0; s < n_samples; ++s) {
    list_start[s] = (uint32_t)at;
    for (int64_t first = 0; first < lanes; first += 64) {
      const int64_t last = first + 64 < lanes ? first + 64 : lanes;
      /* the i-th append of every lane of the group, lane after lane, for i = 0, 1, ... */
      for (int32_t i = 0;; ++i) {
        int any = 0;
        for (int64_t l = first; l < last; ++l) {
          const int32_t v = vertices[s * batch + l / batch];
          const int32_t e = (int32_t)(l % batch) + i * batch;   /* mvsSampling.cu:36 */
          if (e >= degree_of(g, v)) continue;
          any = 1;
          if (rows) { rows[at] = v; cols[at] = g->col[g->row_ptr[v] + e]; }
          at++;
        }
        if (!any) break;
      }
    }
  }
  list_start[n_samples] = (uint32_t)at;
  return at;
}

int64_t ndo_sample_clustergcn(const ndo_graph* g, int64_t n_samples, int n, const int32_t* vertices,
                              int32_t* final_samples, uint32_t* list_start, int32_t* rows, int32_t* cols) {
  const int32_t invalid = g->n_vertices;
  const int64_t F = (int64_t)n + (int64_t)n * n;
  int64_t at = 0;
  for (int64_t s = 0; s < n_samples; ++s) {
    const int32_t* mine = vertices + s * n;
    list_start[s] = (uint32_t)at;
    if (final_samples) {
      for (int64_t i = 0; i < F; ++i) final_samples[s * F + i] = invalid;
      /* step 0: next() returns the transit; it only runs for a transit with edges */
      for (int j = 0; j < n; ++j)
        if (degree_of(g, mine[j]) > 0) final_samples[s * F + j] = mine[j];
    }
    /* step 1: transits are the step-0 outputs */
    for (int j = 0; j < n; ++j) {
      const int32_t v1 = mine[j];
      if (degree_of(g, v1) == 0) continue;
      for (int nbr = 0; nbr < n; ++nbr) {
        const int32_t v2 = mine[nbr];
        if (ndo_has_edge(g, v1, v2)) {               /* clusterGCNSampling.cu:49-57 */
          if (rows) { rows[at] = v1; cols[at] = v2; }
          at++;
        }
      }
    }
  }
  list_start[n_samples] = (uint32_t)at;
  return at;
}
