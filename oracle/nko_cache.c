/* Test infrastructure (CPU oracle): the contact cache that seeds each solve with the previous step's impulses.
 * Restates ContactWarmStart (src/phi/backend_cuda/ops/assemble_rows.cu:1393-1455) with its index
 * (ops/contact_cache.cuh:167-284, 286-338), the row seeding (assemble_rows.cu:1229-1272), the cache rebuild
 * (:1313-1391) and the slot material key (:88-105, 620-622).  Phase 0 runs between AssembleRows and the solve,
 * phase 1 after it; decay_steps is 2 (src/nk/pipeline/pipeline.cpp:905).  The reference finds equal keys through a
 * hash table; here each environment's few entries are compared directly, which selects the same first entry and the
 * same lowest warm point per key. */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "nko_internal.h"

#define NONE 0xffffffffu
static const uint32_t kDecaySteps = 2u;

static uint64_t profile_word(uint64_t hash, uint32_t word) { hash ^= (uint64_t)word; hash *= 0x100000001b3ull; return hash; }
static uint32_t bits(float f) { return f2u(f); }

/* HashMergedContactProfile (:88-105) of two default-authored profiles that differ in friction only
 * (scene/contact_filter.hpp:16-31, 72-130: equal priorities and solmix leave every other term at its default), then
 * the contact law for velocity-only laws (:620-622). */
uint64_t nko_contact_material(float mu1, float mu2, uint32_t law) {
    uint64_t h = 0x4e554b4150524f46ull;
    h = profile_word(h, 2u);             /* kContactProfileSchemaVersion */
    h = profile_word(h, 1u);             /* kContactProfileFlagRefsafe */
    h = profile_word(h, bits(mu1)); h = profile_word(h, bits(mu2));
    h = profile_word(h, bits(0.005f)); h = profile_word(h, bits(0.0001f));
    h = profile_word(h, bits(0.02f)); h = profile_word(h, bits(1.0f));
    const float solimp[5] = {0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
    for (int i = 0; i < 5; ++i) h = profile_word(h, bits(solimp[i]));
    h = profile_word(h, bits(0.0f)); h = profile_word(h, bits(0.0f));   /* margin, gap */
    h = profile_word(h, 3u);                                            /* condim */
    if (h == 0u) h = 0x9e3779b97f4a7c15ull;
    if (law == 1u || law == 2u) { h ^= (uint64_t)law; h *= 1099511628211ull; }   /* kContactLawVelocity, Speculative */
    return h;
}

/* The same hash of any merged profile (mu1, mu2, solref[2], solimp[5], margin, gap, condim; no friction slope),
 * then the law word for the velocity and speculative laws and the cone for the compliant law (:620-623) */
uint64_t nko_contact_material_merged(const float merged[12], uint32_t law, uint32_t cone) {
    uint64_t h = 0x4e554b4150524f46ull;
    h = profile_word(h, 2u);
    h = profile_word(h, 1u);
    h = profile_word(h, bits(merged[0])); h = profile_word(h, bits(merged[1]));
    h = profile_word(h, bits(0.005f)); h = profile_word(h, bits(0.0001f));
    for (int i = 2; i < 11; ++i) h = profile_word(h, bits(merged[i]));
    h = profile_word(h, (uint32_t)merged[11]);   /* condim */
    if (h == 0u) h = 0x9e3779b97f4a7c15ull;
    if (law == 1u || law == 2u) { h ^= (uint64_t)law; h *= 1099511628211ull; }
    if (law == 0u) { h ^= (uint64_t)cone; h *= 1099511628211ull; }
    return h;
}

typedef struct { uint64_t pair, feature, material; uint32_t point; int current; } entry;

static int same_key(const entry* a, const entry* b) { return a->pair == b->pair && a->feature == b->feature && a->material == b->material; }

static int row_offsets(const nko_world* w, uint32_t env, uint32_t slot, uint32_t point, uint32_t* normal, uint32_t* t1, uint32_t* t2) {
    const uint32_t S = w->t.slots;
    const uint32_t first = w->ucontact_row_range[((size_t)env * S + slot) * 2u], points = w->ucontact_row_range[((size_t)env * S + slot) * 2u + 1u];
    if (point >= points) return 0;
    *normal = first + point; *t1 = first + points + point; *t2 = first + 2u * points + point;
    return 1;
}

/* BuildIndex (contact_cache.cuh:286-338) and PrepareContactWarmStartKernel (assemble_rows.cu:1229-1272) */
void nko_env_warm_start_prepare(nko_world* w, uint32_t env) {
    const uint32_t S = w->t.slots, P = S * 4u;
    if (P == 0u) return;
    const size_t base = (size_t)env * P;
    entry* list = (entry*)malloc(sizeof(entry) * 2u * P);
    uint32_t count = 0u;
    for (uint32_t i = 0u; i < P; ++i) {
        w->contact_cache_current_owner[base + i] = 0u; w->contact_cache_old_keep[base + i] = 0u; w->contact_cache_match[base + i] = NONE;
        if ((i & 3u) < w->ucontact_count[(size_t)env * S + i / 4u]) {
            entry e = {w->ucontact_id_pair[base + i], w->ucontact_id_feature[base + i], w->contact_material[(size_t)env * S + i / 4u], i, 1};
            list[count++] = e;
        }
    }
    for (uint32_t j = 0u; j < P; ++j)
        if (w->contact_cache_pair[base + j] != 0u) {
            entry e = {w->contact_cache_pair[base + j], w->contact_cache_feature[base + j], w->contact_cache_material[base + j], j, 0};
            list[count++] = e;
        }
    uint32_t owned = 0u, current = 0u, matched = 0u;
    for (uint32_t k = 0u; k < count; ++k) {
        int head = 1;
        for (uint32_t earlier = 0u; earlier < k && head; ++earlier) if (same_key(&list[earlier], &list[k])) head = 0;
        if (list[k].current) {
            uint32_t warm = NONE;   /* lowest cache point of the key that has not decayed */
            if (head)
                for (uint32_t other = 0u; other < count; ++other)
                    if (!list[other].current && same_key(&list[other], &list[k]) && w->contact_cache_age[base + list[other].point] < kDecaySteps &&
                        list[other].point < warm) warm = list[other].point;
            const uint32_t i = list[k].point;
            w->contact_cache_match[base + i] = warm;
            ++current;
            if (warm != NONE) {
                const float* n = w->ucontact_normal + 3u * (base + i);
                const float* o = w->contact_cache_normal + 3u * (base + warm);
                if (n[0] * o[0] + n[1] * o[1] + n[2] * o[2] > 0.25f) ++matched;
            }
            if (head) { w->contact_cache_current_owner[base + i] = 1u; if (i + 1u > owned) owned = i + 1u; }
        } else if (head && kDecaySteps > 1u && w->contact_cache_age[base + list[k].point] < kDecaySteps - 1u) {
            w->contact_cache_old_keep[base + list[k].point] = 1u;
        }
    }
    free(list);
    w->contact_cache_extent[2u * env + 1u] = owned;
    w->contact_warm_start_counts[2u * env] = current; w->contact_warm_start_counts[2u * env + 1u] = matched;
    /* seed the rows of matched points whose normal has kept its side */
    float* lambda = w->lambda;
    for (uint32_t i = 0u; i < P; ++i) {
        const uint32_t match = w->contact_cache_match[base + i];
        if (match == NONE) continue;
        const float* n = w->ucontact_normal + 3u * (base + i);
        const float* o = w->contact_cache_normal + 3u * (base + match);
        if (n[0] * o[0] + n[1] * o[1] + n[2] * o[2] <= 0.25f) continue;
        uint32_t rn, r1, r2;
        if (!row_offsets(w, env, i / 4u, i & 3u, &rn, &r1, &r2)) continue;
        const float* cached = w->contact_cache_lambda + 4u * (base + match);
        float ot1[3], ot2[3], t1[3], t2[3];
        nko_contact_tangent_basis(o, ot1, ot2);
        nko_contact_tangent_basis(n, t1, t2);
        const v3 old = v3_add(v3_scale(v3_make(ot1[0], ot1[1], ot1[2]), cached[1]), v3_scale(v3_make(ot2[0], ot2[1], ot2[2]), cached[2]));
        lambda[rn] = fmaxf(cached[0], 0.0f);
        lambda[r1] = v3_dot(old, v3_make(t1[0], t1[1], t1[2]));
        lambda[r2] = v3_dot(old, v3_make(t2[0], t2[1], t2[2]));
    }
}

/* BuildRanks, CacheExtentKernel (contact_cache.cuh:340-365) and RebuildContactCacheKernel (assemble_rows.cu:1313-1391) */
void nko_env_warm_start_commit(nko_world* w, uint32_t env) {
    const uint32_t S = w->t.slots, P = S * 4u;
    if (P == 0u) return;
    const size_t base = (size_t)env * P;
    uint32_t* extent = w->contact_cache_extent + 2u * env;
    const uint32_t previous = extent[0] == 0u ? P : (extent[0] - 1u < P ? extent[0] - 1u : P);
    /* the retained old entries in point order, copied out before the cache is overwritten */
    uint32_t* old = (uint32_t*)malloc(sizeof(uint32_t) * (P + 1u));
    uint64_t* spair = (uint64_t*)malloc(sizeof(uint64_t) * 3u * (P + 1u));
    float* sfloat = (float*)malloc(sizeof(float) * 7u * (P + 1u));
    uint32_t* sage = (uint32_t*)malloc(sizeof(uint32_t) * (P + 1u));
    uint32_t retained = 0u, unowned = 0u;
    for (uint32_t i = 0u; i < P; ++i) {
        if (w->contact_cache_current_owner[base + i] == 0u) ++unowned;
        if (w->contact_cache_old_keep[base + i] == 0u) continue;
        spair[3u * retained] = w->contact_cache_pair[base + i]; spair[3u * retained + 1u] = w->contact_cache_feature[base + i];
        spair[3u * retained + 2u] = w->contact_cache_material[base + i];
        memcpy(sfloat + 7u * retained, w->contact_cache_lambda + 4u * (base + i), 4u * sizeof(float));
        memcpy(sfloat + 7u * retained + 4u, w->contact_cache_normal + 3u * (base + i), 3u * sizeof(float));
        sage[retained] = w->contact_cache_age[base + i];
        old[retained++] = i;
    }
    uint32_t next = P - unowned + retained;
    if (extent[1] > next) next = extent[1];
    if (next > P) next = P;
    extent[0] = next + 1u;
    extent[1] = previous > next ? previous : next;
    const uint32_t bound = extent[1] < P ? extent[1] : P;
    const nko_row* rows = (const nko_row*)w->urows;
    uint32_t free_rank = 0u;
    for (uint32_t i = 0u; i < P; ++i) {
        const int owner = w->contact_cache_current_owner[base + i] != 0u;
        const uint32_t rank = free_rank;
        if (!owner) ++free_rank;
        if (i >= bound) continue;
        uint32_t rn, r1, r2;
        if (owner && row_offsets(w, env, i / 4u, i & 3u, &rn, &r1, &r2)) {
            (void)rows; (void)r2;
            const uint32_t stride = r1 - rn;
            w->contact_cache_pair[base + i] = w->ucontact_id_pair[base + i];
            w->contact_cache_feature[base + i] = w->ucontact_id_feature[base + i];
            for (uint32_t k = 0u; k < 4u; ++k) w->contact_cache_lambda[4u * (base + i) + k] = k < 3u ? w->lambda[rn + k * stride] : 0.0f;
            memcpy(w->contact_cache_normal + 3u * (base + i), w->ucontact_normal + 3u * (base + i), 3u * sizeof(float));
            w->contact_cache_material[base + i] = w->contact_material[(size_t)env * S + i / 4u];
            w->contact_cache_age[base + i] = 0u;
            continue;
        }
        /* an owner without rows keeps its place in the free count it never entered (its rank is that of the next free point) */
        if (rank < retained) {
            w->contact_cache_pair[base + i] = spair[3u * rank]; w->contact_cache_feature[base + i] = spair[3u * rank + 1u];
            w->contact_cache_material[base + i] = spair[3u * rank + 2u];
            memcpy(w->contact_cache_lambda + 4u * (base + i), sfloat + 7u * rank, 4u * sizeof(float));
            memcpy(w->contact_cache_normal + 3u * (base + i), sfloat + 7u * rank + 4u, 3u * sizeof(float));
            w->contact_cache_age[base + i] = sage[rank] + 1u;
            continue;
        }
        w->contact_cache_pair[base + i] = 0u; w->contact_cache_feature[base + i] = 0u; w->contact_cache_material[base + i] = 0u;
        memset(w->contact_cache_lambda + 4u * (base + i), 0, 4u * sizeof(float));
        memset(w->contact_cache_normal + 3u * (base + i), 0, 3u * sizeof(float));
        w->contact_cache_age[base + i] = 0u;
    }
    free(old); free(spair); free(sfloat); free(sage);
}
