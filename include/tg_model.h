/*
 * Flat parameter layout of the target model, the counterpart of the reference's
 * parameter_layout (model.h:12-37).  Every matrix is [Out][In] row major.  Order:
 *   embedding[vocab][d], positions[context][d],
 *   per layer: ln1_g[d], ln1_b[d], qkv[3d][d], attn_out[d][d], ln2_g[d], ln2_b[d],
 *              mlp_up[ffn][d], mlp_down[d][ffn]
 *   lnf_g[d], lnf_b[d], head[vocab][d]
 * Weight decay applies to the matrices of the blocks and to the head only (cuda/optim.cuh:5-15).
 */
#ifndef TG_MODEL_H
#define TG_MODEL_H
#include "tg_runtime.h"

#define TG_MAX_DEPTH 64

typedef struct TgLayerParameters {
    int64_t ln1_g, ln1_b, qkv, attn_out, ln2_g, ln2_b, mlp_up, mlp_down;
} TgLayerParameters;
typedef struct TgParameterLayout {
    int64_t embedding, positions, lnf_g, lnf_b, head, count;
    TgLayerParameters layers[TG_MAX_DEPTH];
} TgParameterLayout;

static inline TgParameterLayout tg_parameter_layout(const TgModelConfig *c) {
    TgParameterLayout p;
    int64_t n = 0;
    const int64_t d = c->d_model, f = c->ffn;
    int l;
#define TG_TAKE(field, size) ((field) = n, n += (size))
    TG_TAKE(p.embedding, (int64_t)c->vocab * d);
    TG_TAKE(p.positions, (int64_t)c->base.context * d);
    for (l = 0; l < c->base.depth && l < TG_MAX_DEPTH; ++l) {
        TgLayerParameters *b = &p.layers[l];
        TG_TAKE(b->ln1_g, d);
        TG_TAKE(b->ln1_b, d);
        TG_TAKE(b->qkv, 3 * d * d);
        TG_TAKE(b->attn_out, d * d);
        TG_TAKE(b->ln2_g, d);
        TG_TAKE(b->ln2_b, d);
        TG_TAKE(b->mlp_up, f * d);
        TG_TAKE(b->mlp_down, d * f);
    }
    TG_TAKE(p.lnf_g, d);
    TG_TAKE(p.lnf_b, d);
    TG_TAKE(p.head, (int64_t)c->vocab * d);
#undef TG_TAKE
    p.count = n;
    return p;
}
#endif
