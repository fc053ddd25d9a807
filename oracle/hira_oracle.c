/*
 * hira_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, host-only restatement of the reference's CPU algorithms for the
 * range-search hot path (tree build, halfspace tree walk, exact leaf filter) plus
 * closed-form checkers (brute-force range query, fp64 softmax attention).  Only the
 * test-suite, the smoke check and the CPU-baseline leg of the benchmark may link or
 * call this file; the product path (the HIP library) never does.
 *
 * Reference lines each routine follows (paths relative to the reference tree):
 *   hira_oracle_brute_force     tests/test_cpp_kernels.py:32-55 (closed form
 *                               where(s >= th, s*sc, 0)), kernels/cpp/torch_ext_v3.cpp:159-167
 *   hira_oracle_search_v3       kernels/cpp/torch_ext_v3.cpp:149-244
 *   hira_oracle_build_csr       searcher/cpu.py:345-363
 *   hira_oracle_refine_radii    indexer/cpu.py:263-311
 *   hira_oracle_kmeans          indexer/cpu.py:223-261 (faiss.Kmeans is a third-party
 *                               dependency that is not vendored: restated as textbook
 *                               Lloyd; exact centroid parity with faiss is UNPINNED)
 *   hira_oracle_attention       no reference code exists (attention/hira_attention.py:1-3
 *                               is a docstring); closed form softmax(scaling*q.K_S^T) V_S
 *   hira_oracle_group_traffic   counts, for one GQA group, the nodes/keys the v3 walk
 *                               evaluates (union over the group's query heads)
 *
 * Pinning status (what independent evidence each routine is checked against in tests/):
 *   brute_force   numpy einsum closed form; reference C++ v1-v4 (oracle/_ref) on seeded inputs
 *   search_v3     == brute_force on valid trees; == compiled reference v3 on the same
 *                 tree tensors; committed golden fixtures written from the compiled reference
 *   build_csr     numpy argsort(stable)/bincount
 *   refine_radii  numpy closed form + the reference's radius invariant
 *   kmeans        K=1 -> mean, K=n -> points, nearest-centroid optimality, inertia
 *                 monotonicity.  Centroid values vs faiss: parity unpinned.
 *   attention     torch softmax in fp64; full selection == scaled_dot_product_attention
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define HIRA_ORACLE_ABI 1

int hira_oracle_abi_version(void) { return HIRA_ORACLE_ABI; }

/* fp32 dot product; the reduction order is whatever the compiler picks under the
 * flags this file is built with (the reference builds with -ffast-math and an
 * `omp simd` reduction, kernels/cpp/torch_ext_v3.cpp:25-35). */
static inline float dotf(const float* a, const float* b, int64_t D) {
    float s = 0.0f;
#pragma omp simd reduction(+ : s)
    for (int64_t j = 0; j < D; ++j) s += a[j] * b[j];
    return s;
}

static inline double dotd(const float* a, const float* b, int64_t D) {
    double s = 0.0;
    for (int64_t j = 0; j < D; ++j) s += (double)a[j] * (double)b[j];
    return s;
}

/* out (H_q, N) must be zero-filled by the caller (the reference allocates zeros,
 * torch_ext_v3.cpp:146). */
void hira_oracle_brute_force(const float* keys, int64_t H_kv, int64_t N, int64_t D,
                             const float* query, int64_t H_q, const float* th,
                             const float* sc, const int64_t* q2kv, float* out) {
    (void)H_kv;
    for (int64_t qh = 0; qh < H_q; ++qh) {
        const int64_t h = q2kv[qh];
        const float* q = query + qh * D;
        for (int64_t i = 0; i < N; ++i) {
            const float s = dotf(keys + (h * N + i) * D, q, D);
            if (s >= th[qh]) out[qh * N + i] = s * sc[qh];
        }
    }
}

/* Raw fp32 scores (H_q, N): used to pick thresholds between two scores. */
void hira_oracle_scores(const float* keys, int64_t H_kv, int64_t N, int64_t D,
                        const float* query, int64_t H_q, const int64_t* q2kv, float* out) {
    (void)H_kv;
#pragma omp parallel for schedule(static)
    for (int64_t qh = 0; qh < H_q; ++qh) {
        const int64_t h = q2kv[qh];
        const float* q = query + qh * D;
        for (int64_t i = 0; i < N; ++i) out[qh * N + i] = dotf(keys + (h * N + i) * D, q, D);
    }
}

/*
 * Active-parent tree walk.  Level 0 are the keys, level num_levels-1 the root.
 *   level_centers[l] : (H_kv, K_l, D)   (level 0 entry unused: keys are passed apart)
 *   level_radii[l]   : (H_kv, K_l)
 *   level_offsets[l] : (H_kv, K_{l+1}+1) CSR row starts of the children of level l+1 nodes
 *   level_children[l]: (H_kv, K_l)       child ids at level l, grouped by parent
 * rscale[qh] multiplies the radius in the gate: 1.0 reproduces the reference gate
 * `dot + r >= th` bit for bit; ||q|| gives the bound that is conservative for a
 * non-unit query (searcher/cpu.py:61-63).
 * stats (may be NULL): (H_q, num_levels+1) int64; [qh][l] = nodes evaluated at level l
 * (l = 0: exact leaf checks), [qh][num_levels] = keys selected.
 * out (H_q, N) must be zero-filled by the caller.
 */
void hira_oracle_search_v3(const float* keys, int64_t H_kv, int64_t N, int64_t D,
                           const float* query, int64_t H_q, const float* th, const float* sc,
                           const float* rscale, const int64_t* q2kv, int64_t num_levels,
                           const float* const* level_centers, const float* const* level_radii,
                           const int64_t* level_sizes, const int64_t* const* level_offsets,
                           const int64_t* const* level_children, float* out, int64_t* stats,
                           int num_threads) {
    (void)H_kv;
#ifdef _OPENMP
    if (num_threads > 0) omp_set_num_threads(num_threads);
#else
    (void)num_threads;
#endif
#pragma omp parallel
    {
        int64_t cap = 1;
        for (int64_t l = 0; l < num_levels; ++l)
            if (level_sizes[l] > cap) cap = level_sizes[l];
        int64_t* active = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
        int64_t* next_active = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);

#pragma omp for schedule(static)
        for (int64_t qh = 0; qh < H_q; ++qh) {
            const int64_t h = q2kv[qh];
            const float t = th[qh];
            const float s_out = sc[qh];
            const float rs = rscale[qh];
            const float* q = query + qh * D;
            int64_t* st = stats ? stats + qh * (num_levels + 1) : NULL;
            if (st) memset(st, 0, sizeof(int64_t) * (size_t)(num_levels + 1));

            if (num_levels == 1) { /* flat exact scan, torch_ext_v3.cpp:159-167 */
                for (int64_t i = 0; i < N; ++i) {
                    const float s = dotf(keys + (h * N + i) * D, q, D);
                    if (s >= t) {
                        out[qh * N + i] = s * s_out;
                        if (st) st[num_levels]++;
                    }
                }
                if (st) st[0] = N;
                continue;
            }

            /* root activation, torch_ext_v3.cpp:170-186 */
            const int64_t root = num_levels - 1;
            const int64_t K_root = level_sizes[root];
            int64_t n_active = 0;
            for (int64_t c = 0; c < K_root; ++c) {
                const float s = dotf(level_centers[root] + (h * K_root + c) * D, q, D);
                const float r = level_radii[root][h * K_root + c];
                if (s + rs * r >= t) active[n_active++] = c;
            }
            if (st) st[root] = K_root;

            /* intermediate levels, torch_ext_v3.cpp:188-218 */
            for (int64_t l = root - 1; l >= 1 && n_active > 0; --l) {
                const int64_t K_child = level_sizes[l];
                const int64_t P = level_sizes[l + 1];
                const int64_t* off = level_offsets[l] + h * (P + 1);
                const int64_t* ch = level_children[l] + h * K_child;
                int64_t n_next = 0;
                for (int64_t a = 0; a < n_active; ++a) {
                    const int64_t p = active[a];
                    for (int64_t e = off[p]; e < off[p + 1]; ++e) {
                        const int64_t c = ch[e];
                        const float s = dotf(level_centers[l] + (h * K_child + c) * D, q, D);
                        const float r = level_radii[l][h * K_child + c];
                        if (st) st[l]++;
                        if (s + rs * r >= t) next_active[n_next++] = c;
                    }
                }
                int64_t* tmp = active;
                active = next_active;
                next_active = tmp;
                n_active = n_next;
            }
            if (n_active == 0) continue;

            /* leaf expansion + exact filter, torch_ext_v3.cpp:224-242 */
            const int64_t P0 = level_sizes[1];
            const int64_t* off0 = level_offsets[0] + h * (P0 + 1);
            const int64_t* ch0 = level_children[0] + h * N;
            for (int64_t a = 0; a < n_active; ++a) {
                const int64_t p = active[a];
                for (int64_t e = off0[p]; e < off0[p + 1]; ++e) {
                    const int64_t i = ch0[e];
                    const float s = dotf(keys + (h * N + i) * D, q, D);
                    if (st) st[0]++;
                    if (s >= t) {
                        out[qh * N + i] = s * s_out;
                        if (st) st[num_levels]++;
                    }
                }
            }
        }
        free(active);
        free(next_active);
    }
}

/*
 * For each KV head: the number of tree nodes per level, candidate keys and selected
 * keys that at least one query head of its group evaluates in the walk above.
 * traffic: (H_kv, num_levels+1) int64, [h][l] = nodes evaluated at level l by any head
 * of the group (l = 0: candidate keys), [h][num_levels] = keys selected by any head.
 */
void hira_oracle_group_traffic(const float* keys, int64_t H_kv, int64_t N, int64_t D,
                               const float* query, int64_t H_q, const float* th,
                               const float* rscale, const int64_t* q2kv, int64_t num_levels,
                               const float* const* level_centers,
                               const float* const* level_radii, const int64_t* level_sizes,
                               const int64_t* const* level_offsets,
                               const int64_t* const* level_children, int64_t* traffic) {
    int64_t total = 0;
    for (int64_t l = 0; l < num_levels; ++l) total += level_sizes[l];
    memset(traffic, 0, sizeof(int64_t) * (size_t)(H_kv * (num_levels + 1)));
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t h = 0; h < H_kv; ++h) {
        uint8_t* seen = (uint8_t*)calloc((size_t)total + (size_t)N, 1);
        uint8_t* sel = seen + total;
        int64_t cap = 1;
        for (int64_t l = 0; l < num_levels; ++l)
            if (level_sizes[l] > cap) cap = level_sizes[l];
        int64_t* active = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
        int64_t* next_active = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
        int64_t* base = (int64_t*)malloc(sizeof(int64_t) * (size_t)num_levels);
        base[0] = 0;
        for (int64_t l = 1; l < num_levels; ++l) base[l] = base[l - 1] + level_sizes[l - 1];

        for (int64_t qh = 0; qh < H_q; ++qh) {
            if (q2kv[qh] != h) continue;
            const float t = th[qh];
            const float rs = rscale[qh];
            const float* q = query + qh * D;
            if (num_levels == 1) {
                for (int64_t i = 0; i < N; ++i) {
                    seen[i] = 1;
                    if (dotf(keys + (h * N + i) * D, q, D) >= t) sel[i] = 1;
                }
                continue;
            }
            const int64_t root = num_levels - 1;
            const int64_t K_root = level_sizes[root];
            int64_t n_active = 0;
            for (int64_t c = 0; c < K_root; ++c) {
                seen[base[root] + c] = 1;
                const float s = dotf(level_centers[root] + (h * K_root + c) * D, q, D);
                if (s + rs * level_radii[root][h * K_root + c] >= t) active[n_active++] = c;
            }
            for (int64_t l = root - 1; l >= 1 && n_active > 0; --l) {
                const int64_t K_child = level_sizes[l];
                const int64_t P = level_sizes[l + 1];
                const int64_t* off = level_offsets[l] + h * (P + 1);
                const int64_t* ch = level_children[l] + h * K_child;
                int64_t n_next = 0;
                for (int64_t a = 0; a < n_active; ++a) {
                    const int64_t p = active[a];
                    for (int64_t e = off[p]; e < off[p + 1]; ++e) {
                        const int64_t c = ch[e];
                        seen[base[l] + c] = 1;
                        const float s = dotf(level_centers[l] + (h * K_child + c) * D, q, D);
                        if (s + rs * level_radii[l][h * K_child + c] >= t)
                            next_active[n_next++] = c;
                    }
                }
                int64_t* tmp = active;
                active = next_active;
                next_active = tmp;
                n_active = n_next;
            }
            if (n_active == 0) continue;
            const int64_t P0 = level_sizes[1];
            const int64_t* off0 = level_offsets[0] + h * (P0 + 1);
            const int64_t* ch0 = level_children[0] + h * N;
            for (int64_t a = 0; a < n_active; ++a) {
                const int64_t p = active[a];
                for (int64_t e = off0[p]; e < off0[p + 1]; ++e) {
                    const int64_t i = ch0[e];
                    seen[i] = 1;
                    if (dotf(keys + (h * N + i) * D, q, D) >= t) sel[i] = 1;
                }
            }
        }
        int64_t* tr = traffic + h * (num_levels + 1);
        for (int64_t l = 0; l < num_levels; ++l) {
            int64_t cnt = 0;
            for (int64_t c = 0; c < level_sizes[l]; ++c) cnt += seen[base[l] + c];
            tr[l] = cnt;
        }
        int64_t cnt = 0;
        for (int64_t i = 0; i < N; ++i) cnt += sel[i];
        tr[num_levels] = cnt;
        free(base);
        free(active);
        free(next_active);
        free(seen);
    }
}

/* Parent -> children adjacency from child2parent for one head: children grouped by
 * parent, ascending child id inside a parent (a stable sort; the reference's argsort is
 * unstable so only the grouping is specified).  offsets has P+1 entries. */
void hira_oracle_build_csr(const int64_t* c2p, int64_t C, int64_t P, int64_t* offsets,
                           int64_t* children) {
    memset(offsets, 0, sizeof(int64_t) * (size_t)(P + 1));
    for (int64_t c = 0; c < C; ++c) offsets[c2p[c] + 1]++;
    for (int64_t p = 0; p < P; ++p) offsets[p + 1] += offsets[p];
    int64_t* cursor = (int64_t*)malloc(sizeof(int64_t) * (size_t)(P > 0 ? P : 1));
    memcpy(cursor, offsets, sizeof(int64_t) * (size_t)P);
    for (int64_t c = 0; c < C; ++c) children[cursor[c2p[c]]++] = c;
    free(cursor);
}

/* r_p = max over children assigned to p of (||c_child - c_p||_2 + r_child); a parent
 * with no child keeps -inf (indexer/cpu.py:286-309).  One head. */
void hira_oracle_refine_radii(const float* child_centers, const float* child_radii,
                              const int64_t* assign, int64_t C, int64_t D,
                              const float* parent_centers, int64_t K, float* parent_radii) {
    for (int64_t p = 0; p < K; ++p) parent_radii[p] = -INFINITY;
    for (int64_t c = 0; c < C; ++c) {
        const int64_t p = assign[c];
        const float* a = child_centers + c * D;
        const float* b = parent_centers + p * D;
        float ss = 0.0f;
        for (int64_t j = 0; j < D; ++j) {
            const float d = a[j] - b[j];
            ss += d * d;
        }
        const float contrib = sqrtf(ss) + child_radii[c];
        if (contrib > parent_radii[p]) parent_radii[p] = contrib;
    }
}

static inline uint64_t splitmix64(uint64_t* s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

/* argmin_c ||x - c||^2 for every point, ties to the lowest centroid id; returns the
 * inertia (sum of squared distances to the assigned centroid). */
static double assign_nearest(const float* x, int64_t n, int64_t d, const float* cent, int64_t K,
                             int64_t* assign) {
    double inertia = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : inertia)
    for (int64_t i = 0; i < n; ++i) {
        const float* xi = x + i * d;
        float best = INFINITY;
        int64_t arg = 0;
        for (int64_t c = 0; c < K; ++c) {
            const float* cc = cent + c * d;
            float ss = 0.0f;
            for (int64_t j = 0; j < d; ++j) {
                const float df = xi[j] - cc[j];
                ss += df * df;
            }
            if (ss < best) {
                best = ss;
                arg = c;
            }
        }
        assign[i] = arg;
        inertia += (double)best;
    }
    return inertia;
}

/*
 * Lloyd k-means for one head: K initial centroids = K distinct points drawn by a seeded
 * partial Fisher-Yates shuffle; `niter` rounds of (assign to nearest, centroid = mean of
 * members; an empty cluster keeps its previous centroid); then one final nearest-centroid
 * assignment against the final centroids, which is what the reference reads back with
 * km.index.search(x, 1) (indexer/cpu.py:249-250), so a centroid may end with no member.
 * inertia_trace (may be NULL) receives niter+1 values: the inertia of each assignment.
 */
void hira_oracle_kmeans(const float* x, int64_t n, int64_t d, int64_t K, int64_t niter,
                        uint64_t seed, float* centroids, int64_t* assign,
                        double* inertia_trace) {
    int64_t* idx = (int64_t*)malloc(sizeof(int64_t) * (size_t)n);
    for (int64_t i = 0; i < n; ++i) idx[i] = i;
    uint64_t s = seed;
    for (int64_t i = 0; i < K; ++i) {
        const int64_t j = i + (int64_t)(splitmix64(&s) % (uint64_t)(n - i));
        const int64_t t = idx[i];
        idx[i] = idx[j];
        idx[j] = t;
        memcpy(centroids + i * d, x + idx[i] * d, sizeof(float) * (size_t)d);
    }
    free(idx);

    double* sum = (double*)malloc(sizeof(double) * (size_t)(K * d));
    int64_t* cnt = (int64_t*)malloc(sizeof(int64_t) * (size_t)K);
    for (int64_t it = 0; it < niter; ++it) {
        const double inertia = assign_nearest(x, n, d, centroids, K, assign);
        if (inertia_trace) inertia_trace[it] = inertia;
        memset(sum, 0, sizeof(double) * (size_t)(K * d));
        memset(cnt, 0, sizeof(int64_t) * (size_t)K);
        for (int64_t i = 0; i < n; ++i) {
            const int64_t c = assign[i];
            cnt[c]++;
            for (int64_t j = 0; j < d; ++j) sum[c * d + j] += (double)x[i * d + j];
        }
        for (int64_t c = 0; c < K; ++c) {
            if (cnt[c] == 0) continue;
            for (int64_t j = 0; j < d; ++j)
                centroids[c * d + j] = (float)(sum[c * d + j] / (double)cnt[c]);
        }
    }
    const double inertia = assign_nearest(x, n, d, centroids, K, assign);
    if (inertia_trace) inertia_trace[niter] = inertia;
    free(sum);
    free(cnt);
}

/*
 * out[qh] = sum_i w_i v_i / sum_i w_i over keys with mask[qh, i] != 0,
 * w_i = exp(scaling[qh] * (q . k_i) - max), everything in fp64.  Empty set -> zeros.
 * out: (H_q, Dv) fp64.
 */
void hira_oracle_attention(const float* keys, const float* values, int64_t H_kv, int64_t N,
                           int64_t D, int64_t Dv, const float* query, int64_t H_q,
                           const float* sc, const int64_t* q2kv, const uint8_t* mask,
                           double* out) {
    (void)H_kv;
#pragma omp parallel for schedule(static)
    for (int64_t qh = 0; qh < H_q; ++qh) {
        const int64_t h = q2kv[qh];
        const float* q = query + qh * D;
        double m = -INFINITY;
        for (int64_t i = 0; i < N; ++i) {
            if (!mask[qh * N + i]) continue;
            const double z = (double)sc[qh] * dotd(keys + (h * N + i) * D, q, D);
            if (z > m) m = z;
        }
        double* o = out + qh * Dv;
        for (int64_t j = 0; j < Dv; ++j) o[j] = 0.0;
        if (m == -INFINITY) continue;
        double l = 0.0;
        for (int64_t i = 0; i < N; ++i) {
            if (!mask[qh * N + i]) continue;
            const double z = (double)sc[qh] * dotd(keys + (h * N + i) * D, q, D);
            const double w = exp(z - m);
            l += w;
            const float* v = values + (h * N + i) * Dv;
            for (int64_t j = 0; j < Dv; ++j) o[j] += w * (double)v[j];
        }
        for (int64_t j = 0; j < Dv; ++j) o[j] /= l;
    }
}
