// The ROCm-only graph rewrite and the two fused layers it produces.
//
// The engine runs a transformer encoder layer as ~45 separate ops (MatMul, Add, Reshape, Permute, MatMul,
// Mul, Add, Softmax, MatMul, ... one AbstractLayerAcc::Forward each: source/tnn/core/default_network.cc:571-631).
// This pass, registered like the engine's own optimizers (source/tnn/optimizer/net_optimizer_manager.h:32-66,
// gated on the device like net_optimizer_insert_int8_reformat.cc:41-45) and run on the instance's private
// copy of the graph, collapses them into
//   RocmFusedLinear    : y = act(x W^T + b) (+ residual)     <- MatMul(weight)+Add(bias) [+GELU] [+Add(residual)]
//                                                               or InnerProduct
//   RocmFusedAttention : ctx = softmax(QK^T*scale + mask)V    <- three projections, head split, MatMul, Mul/Div,
//                        with Q,K,V = x Wqkv^T + bqkv            Add(mask), Softmax, MatMul, head merge
// so that a BERT layer becomes 7 launches.  A sub-graph is only rewritten when every intermediate blob has a
// single reader and is not a model output; anything that does not match is left as it is.
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdlib>
#include <functional>

#include "rocm_device.h"

namespace TNN_NS {

namespace {

struct GraphIndex {
    std::map<std::string, int> producer;
    std::map<std::string, std::vector<int>> consumers;
    explicit GraphIndex(const std::vector<std::shared_ptr<LayerInfo>> &layers) {
        for (int i = 0; i < (int)layers.size(); ++i) {
            if (!layers[i])
                continue;
            for (auto &o : layers[i]->outputs)
                producer[o] = i;
            for (auto &in : layers[i]->inputs)
                consumers[in].push_back(i);
        }
    }
    int sole_consumer(const std::string &blob) const {
        auto it = consumers.find(blob);
        return (it == consumers.end() || it->second.size() != 1) ? -1 : it->second[0];
    }
    int producer_of(const std::string &blob) const {
        auto it = producer.find(blob);
        return it == producer.end() ? -1 : it->second;
    }
};

// ---- the attention core, as both rewrites (float and quantised) recognise it --------------------------------------
// Around a Softmax layer:
//   scores = MatMul(q_heads, k_heads^T)            q/k/v_heads <- Permute <- Reshape(head split) <- projection of x
//   [scores * s | scores / s]   (a one-value Mul / Div resource; the same scalar may instead sit on the q or the k^T
//                                operand of the MatMul)
//   [+ mask]                    (either operand order)
//   Softmax over the last axis -> MatMul(probs, v_heads) -> Permute (head merge) -> Reshape
// A chain is only reported when the fused kernel computes exactly what the chain does: every intermediate blob has
// one reader and is no model output, the softmax runs over the keys (its axis parameter is read, not assumed), and the
// additive mask is known -- from the model inputs, the constants and the shape rules of the layers that build it -- to
// hold one value per key and sequence ([B,1,1,S], or [1,1,1,S] / [1,1,S] for every sequence).  Anything else (a
// per-query mask [B,1,S,S], a mask of unknown shape, a softmax over another axis, scores with a second reader) stays
// decomposed and runs through the single-op accs.
struct AttentionCore {
    std::vector<int> chain;         // every layer the fused layer replaces
    std::string mask;               // additive mask blob, empty if there is none
    float scale = 1.0f;             // product of the scalar factors on the scores
    int lq = -1, lk = -1, lv = -1;  // the three projections (whatever the caller's head-split walk accepts as one)
    int rs = -1;                    // the head-merging Reshape: its output is the fused layer's output
    DimsVector split_shape;         // shape parameter of the head-splitting Reshape layers: [.., S, heads, head_dim]
};

class AttentionMatcher {
public:
    // walks `blob` <- Permute(order4 | order3) <- Reshape(head split) <- ... <- projection; returns the projection's
    // layer index or -1, appends the walked layers to the chain and reports the Reshape's shape parameter
    typedef std::function<int(const GraphIndex &, const std::string &, const std::vector<int> &, const std::vector<int> &,
                              std::vector<int> *, DimsVector *)>
        HeadSplitFn;

    AttentionMatcher(NetStructure *s, NetResource *r, HeadSplitFn head_split)
        : structure_(s), resource_(r), head_split_(std::move(head_split)) {}

    bool Match(const GraphIndex &g, int si, AttentionCore *m) {
        auto &L = structure_->layers;
        auto sm = L[si];
        if (!sm || sm->type != LAYER_SOFTMAX || sm->inputs.size() != 1 || sm->outputs.size() != 1)
            return false;
        auto sp = dynamic_cast<SoftmaxLayerParam *>(sm->param.get());
        if (!sp)
            return false;
        m->chain = {si};
        // ---- upstream of the softmax: [Add(mask)] <- [Mul|Div(scalar)] <- MatMul(q, k^T)
        std::string cur = sm->inputs[0];
        bool have_scale = false;
        int qk = -1;
        for (int step = 0; step < 3 && qk < 0; ++step) {
            int pi = g.producer_of(cur);
            if (pi < 0 || !L[pi] || g.sole_consumer(cur) < 0 || IsModelOutput(cur))
                break;
            auto pl = L[pi];
            float v = 0.f;
            if (pl->type == LAYER_ADD && pl->inputs.size() == 2 && m->mask.empty() && !have_scale && !pl->param->quantized &&
                !Res<EltwiseLayerResource>(pl->name)) {
                // scores + mask in either order: the operand that comes out of the score chain is the scores
                bool first_is_scores = IsScoreChain(g, pl->inputs[0]), second_is_scores = IsScoreChain(g, pl->inputs[1]);
                if (first_is_scores == second_is_scores)
                    break;
                m->mask = first_is_scores ? pl->inputs[1] : pl->inputs[0];
                cur     = first_is_scores ? pl->inputs[0] : pl->inputs[1];
                m->chain.push_back(pi);
            } else if (!have_scale && ScalarFactor(pl, &v)) {
                m->scale *= v;
                have_scale = true;
                cur        = pl->inputs[0];
                m->chain.push_back(pi);
            } else if (pl->type == LAYER_MATMUL && pl->inputs.size() == 2 && !Res<MatMulLayerResource>(pl->name)) {
                qk = pi;
                m->chain.push_back(pi);
            } else {
                break;
            }
        }
        if (qk < 0)
            return false;
        // ---- q and k^T operands, each possibly behind a scalar factor of its own (q * s, k^T * sqrt(s) ...)
        DimsVector shape_k, shape_v;
        std::string qb = SkipScalar(g, L[qk]->inputs[0], m), kb = SkipScalar(g, L[qk]->inputs[1], m);
        m->lq = head_split_(g, qb, {0, 2, 1, 3}, {1, 0, 2}, &m->chain, &m->split_shape);
        m->lk = head_split_(g, kb, {0, 2, 3, 1}, {1, 2, 0}, &m->chain, &shape_k);
        if (m->lq < 0 || m->lk < 0)
            return false;
        // the softmax must run over the keys, i.e. the last axis of the scores, whose rank is the head split's
        // (axis normalisation of cpu_softmax_layer_acc.cc:43-44)
        const int rank = (int)m->split_shape.size();
        if (rank < 3 || ((sp->axis % rank) + rank) % rank != rank - 1)
            return false;
        // ---- downstream: MatMul(probs, v) -> Permute -> Reshape
        int pv = g.sole_consumer(sm->outputs[0]);
        if (pv < 0 || !L[pv] || L[pv]->type != LAYER_MATMUL || L[pv]->inputs.size() != 2 || L[pv]->inputs[0] != sm->outputs[0] ||
            L[pv]->inputs[1] == sm->outputs[0] || IsModelOutput(sm->outputs[0]) || Res<MatMulLayerResource>(L[pv]->name))
            return false;
        m->chain.push_back(pv);
        m->lv = head_split_(g, L[pv]->inputs[1], {0, 2, 1, 3}, {1, 0, 2}, &m->chain, &shape_v);
        if (m->lv < 0 || m->split_shape != shape_k || m->split_shape != shape_v)
            return false;
        int pm = g.sole_consumer(L[pv]->outputs[0]);
        if (pm < 0 || !L[pm] || L[pm]->type != LAYER_PERMUTE || IsModelOutput(L[pv]->outputs[0]))
            return false;
        auto pmp = dynamic_cast<PermuteLayerParam *>(L[pm]->param.get());
        if (!pmp || pmp->orders != (rank == 4 ? std::vector<int>{0, 2, 1, 3} : std::vector<int>{1, 0, 2}))
            return false;
        int rs = g.sole_consumer(L[pm]->outputs[0]);
        if (rs < 0 || !L[rs] || L[rs]->type != LAYER_RESHAPE || L[rs]->inputs.size() != 1 || IsModelOutput(L[pm]->outputs[0]))
            return false;
        // the merge must put the heads of one token side by side again: [B, S, hidden] or [tokens, hidden]
        auto rsp = dynamic_cast<ReshapeLayerParam *>(L[rs]->param.get());
        const int hidden = m->split_shape[rank - 2] * m->split_shape[rank - 1];
        if (!rsp || rsp->axis != 0 || rsp->shape.empty() || rsp->shape.back() != hidden)
            return false;
        m->chain.push_back(pm);
        m->chain.push_back(rs);
        m->rs = rs;
        if (L[m->lq]->inputs[0] != L[m->lk]->inputs[0] || L[m->lq]->inputs[0] != L[m->lv]->inputs[0])
            return false;
        // ---- the mask: computed before the chain starts, and one value per key
        if (!m->mask.empty()) {
            int first = *std::min_element(m->chain.begin(), m->chain.end());
            int pmask = g.producer_of(m->mask);
            bool early = pmask >= 0 ? pmask < first
                                    : structure_->inputs_shape_map.count(m->mask) > 0 || resource_->constant_map.count(m->mask) > 0;
            DimsVector md;
            if (!early || !StaticDims(g, m->mask, &md, 0) || (int)md.size() != rank)
                return false;
            for (int a = 1; a + 1 < rank; ++a)
                if (md[a] != 1)
                    return false;  // a per-head or per-query mask
            if (rank == 3 && md[0] != 1)
                return false;  // [B*heads, 1, S]: one row per (sequence, head)
        }
        return true;
    }

private:
    bool IsModelOutput(const std::string &b) const { return structure_->outputs.count(b) > 0; }
    template <typename T> T *Res(const std::string &name) const {
        auto it = resource_->resource_map.find(name);
        return it == resource_->resource_map.end() ? nullptr : dynamic_cast<T *>(it->second.get());
    }
    // Mul / Div by one fp32 value held in the layer's resource: *factor is what it multiplies its input by
    bool ScalarFactor(const std::shared_ptr<LayerInfo> &l, float *factor) const {
        if (!l || (l->type != LAYER_MUL && l->type != LAYER_DIV) || l->inputs.size() != 1 || l->param->quantized)
            return false;
        auto er = Res<EltwiseLayerResource>(l->name);
        if (!er || er->element_handle.GetDataCount() != 1 || er->element_handle.GetDataType() != DATA_TYPE_FLOAT)
            return false;
        auto bp = dynamic_cast<MultidirBroadcastLayerParam *>(l->param.get());
        float v = er->element_handle.force_to<float *>()[0];
        if (l->type == LAYER_DIV && bp && bp->weight_input_index == 0)
            return false;  // s / scores is no scaling
        *factor = l->type == LAYER_MUL ? v : 1.0f / v;
        return true;
    }
    // does `blob` come out of MatMul(2 inputs), possibly through one scalar factor?
    bool IsScoreChain(const GraphIndex &g, const std::string &blob) const {
        auto &L = structure_->layers;
        int p   = g.producer_of(blob);
        float v;
        if (p >= 0 && L[p] && ScalarFactor(L[p], &v))
            p = g.producer_of(L[p]->inputs[0]);
        return p >= 0 && L[p] && L[p]->type == LAYER_MATMUL && L[p]->inputs.size() == 2;
    }
    // a scalar factor on an operand of the score MatMul is folded into the scale
    std::string SkipScalar(const GraphIndex &g, const std::string &blob, AttentionCore *m) const {
        auto &L = structure_->layers;
        int p   = g.producer_of(blob);
        float v;
        if (p < 0 || !L[p] || !ScalarFactor(L[p], &v) || g.sole_consumer(blob) < 0 || IsModelOutput(blob))
            return blob;
        m->scale *= v;
        m->chain.push_back(p);
        return L[p]->inputs[0];
    }
    // The dims of `blob` as far as the graph fixes them before any shape inference has run: model inputs, constants,
    // and what Cast / Unsqueeze / Squeeze / Reshape(static) / element-wise layers make of them.  false = unknown.
    bool StaticDims(const GraphIndex &g, const std::string &blob, DimsVector *dims, int depth) const {
        if (depth > 8)
            return false;
        auto in = structure_->inputs_shape_map.find(blob);
        if (in != structure_->inputs_shape_map.end()) {
            *dims = in->second;
            return true;
        }
        auto ct = resource_->constant_map.find(blob);
        if (ct != resource_->constant_map.end() && ct->second) {
            *dims = ct->second->GetBufferDims();
            return !dims->empty();
        }
        auto &L = structure_->layers;
        int p   = g.producer_of(blob);
        if (p < 0 || !L[p] || L[p]->outputs.size() != 1)
            return false;
        auto l = L[p];
        switch (l->type) {
            case LAYER_CAST:
                return l->inputs.size() == 1 && StaticDims(g, l->inputs[0], dims, depth + 1);
            case LAYER_UNSQUEEZE: {  // unsqueeze_layer.cc:44-54
                auto sp = dynamic_cast<SqueezeLayerParam *>(l->param.get());
                if (!sp || l->inputs.size() != 1 || !StaticDims(g, l->inputs[0], dims, depth + 1))
                    return false;
                for (int axis : sp->axes) {
                    axis = axis < 0 ? axis + (int)dims->size() + 1 : axis;
                    if (axis < 0 || axis > (int)dims->size())
                        return false;
                    dims->insert(dims->begin() + axis, 1);
                }
                return true;
            }
            case LAYER_ADD:
            case LAYER_SUB:
            case LAYER_MUL:
            case LAYER_DIV: {
                // element-wise with broadcasting (multidir_broadcast_layer.cc:59-111): the extent of each axis is the
                // largest among the operands, shorter shapes are padded in front
                std::vector<DimsVector> ops;
                for (auto &i : l->inputs) {
                    DimsVector d;
                    if (!StaticDims(g, i, &d, depth + 1))
                        return false;
                    ops.push_back(d);
                }
                if (auto er = Res<EltwiseLayerResource>(l->name)) {
                    DimsVector d = er->element_handle.GetBufferDims();
                    if (er->element_handle.GetDataCount() == 1)
                        d = {1};
                    if (d.empty())
                        return false;
                    ops.push_back(d);
                }
                if (ops.empty())
                    return false;
                size_t rank = 0;
                for (auto &d : ops)
                    rank = std::max(rank, d.size());
                dims->assign(rank, 1);
                for (auto &d : ops)
                    for (size_t a = 0; a < d.size(); ++a) {
                        int &o = (*dims)[rank - d.size() + a];
                        if (d[a] != 1 && o != 1 && d[a] != o)
                            return false;
                        o = std::max(o, d[a]);
                    }
                return true;
            }
            default:
                return false;
        }
    }

    NetStructure *structure_;
    NetResource *resource_;
    HeadSplitFn head_split_;
};

// What the passes below take for granted when they index a layer's blob lists and read weights by the dims written
// next to them, checked once per pass: a model file that breaks one of these (a layer of the path without input or
// output, a weight record whose dims promise more elements than it holds) is reported as an invalid model here instead
// of being read out of bounds further down.
static Status RocmCheckModel(NetStructure *s, NetResource *r) {
    for (auto &l : s->layers) {
        if (!l || !l->param)
            return Status(TNNERR_INVALID_MODEL, "a layer record is empty");
        if (l->outputs.empty())
            return Status(TNNERR_INVALID_MODEL, "layer " + l->name + " has no output blob");
        switch (l->type) {
            case LAYER_MATMUL: case LAYER_INNER_PRODUCT: case LAYER_ADD: case LAYER_SUB: case LAYER_MUL: case LAYER_DIV:
            case LAYER_SOFTMAX: case LAYER_PERMUTE: case LAYER_RESHAPE: case LAYER_LAYER_NORM: case LAYER_GELU:
            case LAYER_REFORMAT: case LAYER_CAST: case LAYER_UNSQUEEZE: case LAYER_SQUEEZE: case LAYER_TANH:
                if (l->inputs.empty())
                    return Status(TNNERR_INVALID_MODEL, "layer " + l->name + " has no input blob");
                break;
            default: break;
        }
    }
    auto holds = [](const RawBuffer &b) {
        const DimsVector d = b.GetBufferDims();
        if (d.empty())
            return true;  // records of the first file version carry no dims
        long n = 1;
        for (int v : d) {
            if (v < 0 || (n *= v) > (1L << 31))
                return false;
        }
        return n == (long)b.GetDataCount();
    };
    auto bad = [](const std::string &owner, const char *what) {
        return Status(TNNERR_INVALID_MODEL, "resource of " + owner + ": the dims of " + what + " do not match its data");
    };
    for (auto &kv : r->resource_map) {
        LayerResource *res = kv.second.get();
        if (auto m = dynamic_cast<MatMulLayerResource *>(res)) {
            if (!holds(m->weight))
                return bad(kv.first, "the weight");
        } else if (auto ip = dynamic_cast<InnerProductLayerResource *>(res)) {
            if (!holds(ip->weight_handle) || !holds(ip->bias_handle) || !holds(ip->scale_handle))
                return bad(kv.first, "weight, bias or scale");
        } else if (auto e = dynamic_cast<EltwiseLayerResource *>(res)) {
            if (!holds(e->element_handle))
                return bad(kv.first, "the operand");
        } else if (auto g = dynamic_cast<GatherLayerResource *>(res)) {
            if (!holds(g->data) || !holds(g->indices))
                return bad(kv.first, "data or indices");
        } else if (auto q = dynamic_cast<IntScaleResource *>(res)) {
            if (!holds(q->scale_handle) || !holds(q->bias_handle))
                return bad(kv.first, "scale or bias");
        }
    }
    for (auto &kv : r->constant_map)
        if (kv.second && !holds(*kv.second))
            return bad(kv.first, "the constant");
    return TNN_OK;
}

// Weights a model file stores in half precision (the converter's option for files of half the size) are widened to fp32
// records before the rewrites look at them: the rewrites fold, transpose and concatenate weights in fp32, and the CPU
// devices widen them as well, layer by layer (ConvertHalfResource, cpu_layer_acc.h:70-82, x86_mat_mul_layer_acc.cc:36-40).
// Exact: every half value is an fp32 value.
static float RocmHalfBitsToFloat(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                ++shift;
            }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
static void RocmWidenHalfRecord(RawBuffer &b) {
    if (b.GetDataType() != DATA_TYPE_HALF || b.GetBytesSize() <= 0)
        return;
    const int count = b.GetDataCount();
    RawBuffer wide(count * 4, b.GetBufferDims());
    wide.SetDataType(DATA_TYPE_FLOAT);
    const uint16_t *src = b.force_to<uint16_t *>();
    float *dst          = wide.force_to<float *>();
    for (int i = 0; i < count; ++i)
        dst[i] = RocmHalfBitsToFloat(src[i]);
    b = wide;
}
static void RocmWidenHalfWeights(NetResource *r) {
    for (auto &kv : r->resource_map) {
        LayerResource *res = kv.second.get();
        if (auto m = dynamic_cast<MatMulLayerResource *>(res)) {
            RocmWidenHalfRecord(m->weight);
        } else if (auto ip = dynamic_cast<InnerProductLayerResource *>(res)) {
            RocmWidenHalfRecord(ip->weight_handle);
            RocmWidenHalfRecord(ip->bias_handle);
        } else if (auto e = dynamic_cast<EltwiseLayerResource *>(res)) {
            RocmWidenHalfRecord(e->element_handle);
        } else if (auto g = dynamic_cast<GatherLayerResource *>(res)) {
            RocmWidenHalfRecord(g->data);
        }
    }
    for (auto &kv : r->constant_map)
        if (kv.second)
            RocmWidenHalfRecord(*kv.second);
}

class RocmFusionPass : public optimizer::NetOptimizer {
public:
    std::string Strategy() override { return "net_optimizer_rocm_fuse_encoder"; }
    bool IsSupported(const NetworkConfig &c) override {
        half_ = c.precision != PRECISION_HIGH;
        return c.device_type == DEVICE_ROCM;
    }

    Status Optimize(NetStructure *s, NetResource *r) override {
        RETURN_ON_NEQ(RocmCheckModel(s, r), TNN_OK);
        RocmWidenHalfWeights(r);
        structure_ = s;
        resource_  = r;
        FuseEmbedding();
        FuseLinear();
        FoldGelu();
        FoldResidual();
        if (half_)
            FuseAttention();  // the attention kernel computes in fp16; fp32 nets keep the decomposed core
        const char *fold = getenv("TNN_ROCM_FOLD_LN");
        if (half_ && !(fold && fold[0] == '0'))
            FoldLayerNorm();
        const char *hand = getenv("TNN_ROCM_LN_STATS");  // "0" keeps the LayerNorm output of a folding layer a tensor
        if (half_ && !(fold && fold[0] == '0') && !(hand && hand[0] == '0')) {
            HandOverRowStatistics();
            const char *sums = getenv("TNN_ROCM_LN_SUMS");  // "0": folding layers take the statistics from their A tiles
            if (!(sums && sums[0] == '0'))
                HandOverRowSums();
        }
        return TNN_OK;
    }

private:
    bool IsModelOutput(const std::string &b) const { return structure_->outputs.count(b) > 0; }
    void Compact() {
        auto &L = structure_->layers;
        L.erase(std::remove(L.begin(), L.end(), nullptr), L.end());
    }
    template <typename T> T *ParamOf(const std::shared_ptr<LayerInfo> &l) { return dynamic_cast<T *>(l->param.get()); }
    template <typename T> T *ResOf(const std::string &name) {
        auto it = resource_->resource_map.find(name);
        return it == resource_->resource_map.end() ? nullptr : dynamic_cast<T *>(it->second.get());
    }

    std::shared_ptr<LayerInfo> MakeLinear(const std::string &name, const std::string &in, const std::string &out, int N,
                                          int K, const float *w_nk_or_null, const float *w_kn_or_null, const float *bias,
                                          bool has_bias) {
        auto l       = std::make_shared<LayerInfo>();
        l->type      = LAYER_ROCM_FUSED_LINEAR;
        l->type_str  = "RocmFusedLinear";
        l->name      = name;
        l->inputs    = {in};
        l->outputs   = {out};
        auto p       = std::make_shared<RocmFusedLinearParam>();
        p->type      = l->type_str;
        p->name      = name;
        p->num_output = N;
        p->has_bias  = has_bias ? 1 : 0;
        l->param     = p;
        auto res     = std::make_shared<RocmFusedLinearResource>();
        res->name    = name;
        res->weight_nk = RawBuffer(N * K * 4, {N, K});
        float *w     = res->weight_nk.force_to<float *>();
        if (w_nk_or_null) {
            memcpy(w, w_nk_or_null, (size_t)N * K * 4);
        } else {
            for (int k = 0; k < K; ++k)
                for (int n = 0; n < N; ++n)
                    w[(size_t)n * K + k] = w_kn_or_null[(size_t)k * N + n];
        }
        if (has_bias) {
            res->bias = RawBuffer(N * 4, {N});
            memcpy(res->bias.force_to<float *>(), bias, (size_t)N * 4);
        }
        resource_->resource_map[name] = res;
        return l;
    }

    // Gather(word table, ids) -> Add(position constant [S,H]) -> Add(Gather(type table, type ids)) -> LayerNorm
    //                                                                                   ==> RocmFusedEmbedding
    void FuseEmbedding() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        auto table_gather = [&](int i) -> GatherLayerResource * {
            if (i < 0 || !L[i] || L[i]->type != LAYER_GATHER || L[i]->inputs.size() != 1)
                return nullptr;
            auto gp = ParamOf<GatherLayerParam>(L[i]);
            auto gr = ResOf<GatherLayerResource>(L[i]->name);
            if (!gp || !gr || gp->axis != 0 || !gp->data_in_resource || gp->indices_in_resource ||
                gr->data.GetBufferDims().size() != 2 || gr->data.GetDataType() != DATA_TYPE_FLOAT)
                return nullptr;
            return gr;
        };
        for (int li = 0; li < (int)L.size(); ++li) {
            auto ln = L[li];
            if (!ln || ln->type != LAYER_LAYER_NORM || ln->inputs.size() != 3 || ln->outputs.size() != 1)
                continue;
            int ai = g.producer_of(ln->inputs[0]);  // Add(word + pos, type)
            if (ai < 0 || !L[ai] || L[ai]->type != LAYER_ADD || L[ai]->inputs.size() != 2 || g.sole_consumer(ln->inputs[0]) != li ||
                IsModelOutput(ln->inputs[0]) || ResOf<EltwiseLayerResource>(L[ai]->name))
                continue;
            // the inner Add is either Add(word gather, position constant) or Add(word gather, position gather)
            int pi = -1, ti = -1;
            for (int side = 0; side < 2 && pi < 0; ++side) {
                int a = g.producer_of(L[ai]->inputs[side]), b = g.producer_of(L[ai]->inputs[1 - side]);
                if (a >= 0 && L[a] && L[a]->type == LAYER_ADD && table_gather(b) &&
                    (L[a]->inputs.size() == 1 ||
                     (L[a]->inputs.size() == 2 && !ResOf<EltwiseLayerResource>(L[a]->name) &&
                      table_gather(g.producer_of(L[a]->inputs[0])) && table_gather(g.producer_of(L[a]->inputs[1])))))
                    pi = a, ti = b;
            }
            if (pi < 0)
                continue;
            const bool pos_gather = L[pi]->inputs.size() == 2;
            auto pos = ResOf<EltwiseLayerResource>(L[pi]->name);
            int wi   = g.producer_of(L[pi]->inputs[0]);
            int pgi  = pos_gather ? g.producer_of(L[pi]->inputs[1]) : -1;  // fp32 a+b == b+a: either may be "word"
            auto wr = table_gather(wi), tr = table_gather(ti);
            auto pgr = pos_gather ? table_gather(pgi) : nullptr;
            if (pgr && wr && pgr->data.GetBufferDims()[0] > wr->data.GetBufferDims()[0]) {
                std::swap(wi, pgi);  // the vocabulary is the larger table; its ids carry the [B,S] shape
                std::swap(wr, pgr);
            }
            if (!wr || !tr || (pos_gather ? !pgr : (!pos || pos->element_handle.GetDataType() != DATA_TYPE_FLOAT)))
                continue;
            const int H = wr->data.GetBufferDims()[1];
            if (tr->data.GetBufferDims()[1] != H)
                continue;
            if (pos_gather) {
                if (pgr->data.GetBufferDims()[1] != H)
                    continue;
            } else {
                auto pd = pos->element_handle.GetBufferDims();
                if (pd.size() < 2 || pd.back() != H || pos->element_handle.GetDataCount() != pd[pd.size() - 2] * H)
                    continue;  // the constant must be one [S,H] matrix (leading dimensions of extent 1)
            }
            bool single = true;
            for (int idx : {pi, ti, wi, pgi})
                if (idx >= 0)
                    single &= g.sole_consumer(L[idx]->outputs[0]) >= 0 && !IsModelOutput(L[idx]->outputs[0]);
            if (!single)
                continue;
            auto lp      = ParamOf<LayerNormLayerParam>(ln);
            auto fl      = std::make_shared<LayerInfo>();
            fl->type     = LAYER_ROCM_FUSED_EMBEDDING;
            fl->type_str = "RocmFusedEmbedding";
            fl->name     = ln->name + "_fused_embedding";
            fl->inputs   = {L[wi]->inputs[0], L[ti]->inputs[0], ln->inputs[1], ln->inputs[2]};
            if (pos_gather)
                fl->inputs.push_back(L[pgi]->inputs[0]);  // fifth input: the position ids
            fl->outputs  = ln->outputs;
            auto fp      = std::make_shared<RocmFusedEmbeddingParam>();
            fp->type     = fl->type_str;
            fp->name     = fl->name;
            fp->eps      = lp->eps;
            fl->param    = fp;
            auto fr      = std::make_shared<RocmFusedEmbeddingResource>();
            fr->name     = fl->name;
            fr->word     = wr->data;
            fr->type     = tr->data;
            fr->pos      = pos_gather ? pgr->data : pos->element_handle;
            resource_->resource_map[fl->name] = fr;
            L[wi] = L[ti] = L[pi] = L[ai] = nullptr;
            if (pos_gather)
                L[pgi] = nullptr;
            // the fused layer goes where the LayerNorm was: every input (ids, constants) exists before that point
            L[li] = fl;
        }
        Compact();
    }

    // MatMul(weight_position=1, fp32 [K,N] resource) -> Add(bias resource of N values)   ==> RocmFusedLinear
    // InnerProduct (float, axis = last)                                                 ==> RocmFusedLinear
    void FuseLinear() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            auto l = L[i];
            if (!l)
                continue;
            if (l->type == LAYER_MATMUL && l->inputs.size() == 1) {
                auto mp = ParamOf<MatMulLayerParam>(l);
                auto mr = ResOf<MatMulLayerResource>(l->name);
                if (!mp || !mr || mp->weight_position != 1 || mr->weight.GetDataType() != DATA_TYPE_FLOAT)
                    continue;
                auto wd = mr->weight.GetBufferDims();
                if (wd.size() != 2)
                    continue;
                int K = wd[0], N = wd[1];
                if (K <= 0 || N <= 0 || (long)K * N != (long)mr->weight.GetDataCount())
                    continue;
                const std::string &mid = l->outputs[0];
                int j = g.sole_consumer(mid);
                const float *bias = nullptr;
                std::string out   = mid;
                if (j > i && L[j] && L[j]->type == LAYER_ADD && L[j]->inputs.size() == 1 && !IsModelOutput(mid)) {
                    auto ar = ResOf<EltwiseLayerResource>(L[j]->name);
                    if (ar && ar->element_handle.GetDataType() == DATA_TYPE_FLOAT && ar->element_handle.GetDataCount() == N) {
                        auto ad = ar->element_handle.GetBufferDims();
                        if (ad.empty() || ad.back() == N) {  // a vector over the last axis
                            bias = ar->element_handle.force_to<float *>();
                            out  = L[j]->outputs[0];
                        }
                    }
                }
                auto fused = MakeLinear(l->name + "_fused", l->inputs[0], out, N, K, nullptr,
                                        mr->weight.force_to<float *>(), bias, bias != nullptr);
                L[i] = fused;
                if (bias)
                    L[j] = nullptr;
            } else if (l->type == LAYER_INNER_PRODUCT && !l->param->quantized) {
                auto ip = ParamOf<InnerProductLayerParam>(l);
                auto ir = ResOf<InnerProductLayerResource>(l->name);
                if (!ip || !ir || ir->weight_handle.GetDataType() != DATA_TYPE_FLOAT || ip->transpose != 0)
                    continue;
                int N = ip->num_output;
                if (N <= 0 || ir->weight_handle.GetDataCount() % N != 0)
                    continue;
                int K = ir->weight_handle.GetDataCount() / N;
                // only the "last axis" form is a row-wise linear map; shapes are not known here, so require the
                // usual exported forms axis = 1 on [T,K] blobs (checked again by the layer's shape inference)
                if (ip->axis != 1)
                    continue;
                bool hb = ip->has_bias && ir->bias_handle.GetDataCount() == N &&
                          ir->bias_handle.GetDataType() == DATA_TYPE_FLOAT;
                if (ip->has_bias && !hb && ir->bias_handle.GetDataCount() > 0)
                    continue;  // a bias of another type or length: leave the layer to its un-fused acc
                auto fused = MakeLinear(l->name + "_fused", l->inputs[0], l->outputs[0], N, K,
                                        ir->weight_handle.force_to<float *>(), nullptr,
                                        hb ? ir->bias_handle.force_to<float *>() : nullptr, hb);
                ParamOf<RocmFusedLinearParam>(fused)->axis = ip->axis;
                L[i] = fused;
            }
        }
        Compact();
    }

    void FoldGelu() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            auto l = L[i];
            if (!l || l->type != LAYER_ROCM_FUSED_LINEAR)
                continue;
            int j = g.sole_consumer(l->outputs[0]);
            if (j > i && L[j] && L[j]->type == LAYER_GELU && !IsModelOutput(l->outputs[0])) {
                ParamOf<RocmFusedLinearParam>(l)->gelu = 1;
                l->outputs[0]                           = L[j]->outputs[0];
                L[j]                                    = nullptr;
            }
        }
        Compact();
    }

    void FoldResidual() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            auto l = L[i];
            if (!l || l->type != LAYER_ROCM_FUSED_LINEAR)
                continue;
            auto p = ParamOf<RocmFusedLinearParam>(l);
            if (p->gelu || p->has_residual || IsModelOutput(l->outputs[0]))
                continue;
            int j = g.sole_consumer(l->outputs[0]);
            if (j <= i || !L[j] || L[j]->type != LAYER_ADD || L[j]->inputs.size() != 2 || L[j]->param->quantized ||
                ResOf<EltwiseLayerResource>(L[j]->name))
                continue;
            const std::string &other = L[j]->inputs[0] == l->outputs[0] ? L[j]->inputs[1] : L[j]->inputs[0];
            if (other == l->outputs[0])
                continue;
            int po = g.producer_of(other);
            bool available = po >= 0 ? po < i : structure_->inputs_shape_map.count(other) > 0;
            if (!available)
                continue;
            // the residual must have the linear's output shape; the layer's Init re-checks this
            p->has_residual = 1;
            l->inputs.push_back(other);
            l->outputs[0] = L[j]->outputs[0];
            L[j]          = nullptr;
        }
        Compact();
    }

    // follow `blob` back through Reshape(-> rank 3/4 head split) and Permute(order) to a fused linear on x
    int HeadSplitSource(const GraphIndex &g, const std::string &blob, const std::vector<int> &order4,
                        const std::vector<int> &order3, std::vector<int> *chain, DimsVector *split_shape) {
        auto &L = structure_->layers;
        int pi  = g.producer_of(blob);
        if (pi < 0 || !L[pi] || L[pi]->type != LAYER_PERMUTE || g.sole_consumer(blob) < 0 || IsModelOutput(blob))
            return -1;
        auto pp = ParamOf<PermuteLayerParam>(L[pi]);
        if (!pp || (pp->orders != order4 && pp->orders != order3))
            return -1;
        const std::string &rb = L[pi]->inputs[0];
        int ri                = g.producer_of(rb);
        if (ri < 0 || !L[ri] || L[ri]->type != LAYER_RESHAPE || g.sole_consumer(rb) != pi || IsModelOutput(rb))
            return -1;
        auto rp = ParamOf<ReshapeLayerParam>(L[ri]);
        if (!rp || rp->axis != 0 || rp->shape.size() != pp->orders.size() || L[ri]->inputs.size() != 1)
            return -1;
        const std::string &lb = L[ri]->inputs[0];
        int li                = g.producer_of(lb);
        if (li < 0 || !L[li] || L[li]->type != LAYER_ROCM_FUSED_LINEAR || g.sole_consumer(lb) != ri || IsModelOutput(lb))
            return -1;
        auto lp = ParamOf<RocmFusedLinearParam>(L[li]);
        if (lp->gelu || lp->has_residual)
            return -1;
        chain->push_back(pi);
        chain->push_back(ri);
        chain->push_back(li);
        *split_shape = rp->shape;
        return li;
    }

    void FuseAttention() {
        auto &L = structure_->layers;
        bool changed = true;
        while (changed) {
            changed = false;
            GraphIndex g(L);
            for (int si = 0; si < (int)L.size() && !changed; ++si) {
                auto sm = L[si];
                if (!sm || sm->type != LAYER_SOFTMAX)
                    continue;
                AttentionCore m;
                AttentionMatcher matcher(structure_, resource_,
                                         [this](const GraphIndex &gi, const std::string &blob, const std::vector<int> &o4,
                                                const std::vector<int> &o3, std::vector<int> *chain, DimsVector *shape) {
                                             return HeadSplitSource(gi, blob, o4, o3, chain, shape);
                                         });
                if (!matcher.Match(g, si, &m))
                    continue;
                const std::vector<int> &chain = m.chain;
                const std::string &mask = m.mask;
                const float scale = m.scale;
                const int lq = m.lq, lk = m.lk, lv = m.lv, rs = m.rs;
                const DimsVector &shape_q = m.split_shape;
                // ---- the three projections are plain linears of equal width
                auto rq = ResOf<RocmFusedLinearResource>(L[lq]->name), rk = ResOf<RocmFusedLinearResource>(L[lk]->name),
                     rv = ResOf<RocmFusedLinearResource>(L[lv]->name);
                if (!rq || !rk || !rv)
                    continue;
                auto dq = rq->weight_nk.GetBufferDims();
                if (dq != rk->weight_nk.GetBufferDims() || dq != rv->weight_nk.GetBufferDims())
                    continue;
                int H = dq[0], K = dq[1];
                int heads    = shape_q[shape_q.size() - 2];
                int head_dim = shape_q.back();
                int seq      = shape_q[shape_q.size() - 3];
                // seq 0 / -1: the split copies (or infers) the sequence length, i.e. the model is meant for
                // Instance::Reshape; the acc then reads S from its input blob [B,S,H] at every reshape
                if (heads * head_dim != H || K != H || head_dim != 64 || seq < -1)
                    continue;
                int first = *std::min_element(chain.begin(), chain.end());
                // ---- build the fused layer
                auto fl      = std::make_shared<LayerInfo>();
                fl->type     = LAYER_ROCM_FUSED_ATTENTION;
                fl->type_str = "RocmFusedAttention";
                fl->name     = sm->name + "_fused_attention";
                fl->inputs   = {L[lq]->inputs[0]};
                if (!mask.empty())
                    fl->inputs.push_back(mask);
                fl->outputs  = {L[rs]->outputs[0]};
                auto fp      = std::make_shared<RocmFusedAttentionParam>();
                fp->type     = fl->type_str;
                fp->name     = fl->name;
                fp->heads    = heads;
                fp->head_dim = head_dim;
                fp->scale    = scale;
                fp->has_mask = mask.empty() ? 0 : 1;
                fp->split_rank  = (int)shape_q.size();
                fp->merge_shape = ParamOf<ReshapeLayerParam>(L[rs])->shape;
                fl->param    = fp;
                fp->seq_len  = seq > 0 ? seq : 0;
                auto fr       = std::make_shared<RocmFusedLinearResource>();
                fr->name      = fl->name;
                fr->weight_nk = RawBuffer(3 * H * K * 4, {3 * H, K});
                fr->bias      = RawBuffer(3 * H * 4, {3 * H});
                RocmFusedLinearResource *src[3] = {rq, rk, rv};
                for (int t = 0; t < 3; ++t) {
                    memcpy(fr->weight_nk.force_to<float *>() + (size_t)t * H * K, src[t]->weight_nk.force_to<float *>(),
                           (size_t)H * K * 4);
                    if (src[t]->bias.GetDataCount() == H)
                        memcpy(fr->bias.force_to<float *>() + (size_t)t * H, src[t]->bias.force_to<float *>(), (size_t)H * 4);
                }
                resource_->resource_map[fl->name] = fr;
                for (int idx : chain)
                    L[idx] = nullptr;
                L[first] = fl;
                changed  = true;
            }
            Compact();
        }
    }

    // LayerNorm(t, gamma, beta -> y) whose output is the A operand of exactly one RocmFusedLinear, or the input of
    // one RocmFusedAttention: that layer reads t instead and applies the normalisation inside its GEMM (see
    // LnFloatEpilogue in the GEMM source); the LayerNorm launch disappears.  If y has other readers (the residual
    // additions) the layer also writes y, as a second output; they must come after it in the layer order.
    // gamma / beta must be constants over the last axis, a multiple of 128 wide.
    void FoldLayerNorm() {
        auto &L = structure_->layers;
        auto constant = [&](const std::string &name, int count) -> RawBuffer * {
            auto it = resource_->constant_map.find(name);
            if (it == resource_->constant_map.end() || !it->second || it->second->GetDataType() != DATA_TYPE_FLOAT ||
                it->second->GetDataCount() != count)
                return nullptr;
            return it->second.get();
        };
        for (int li = 0; li < (int)L.size(); ++li) {
            auto ln = L[li];
            if (!ln || ln->type != LAYER_LAYER_NORM || ln->inputs.size() != 3 || ln->outputs.size() != 1 || ln->param->quantized)
                continue;
            GraphIndex g(L);
            auto lp = ParamOf<LayerNormLayerParam>(ln);
            const std::string t = ln->inputs[0], y = ln->outputs[0];
            auto cit = g.consumers.find(y);
            if (!lp || lp->reduce_dims_size != 1 || cit == g.consumers.end())
                continue;
            int owner = -1, owners = 0, C = 0;
            for (int ci : cit->second) {
                auto c = L[ci];
                if (!c || c->inputs[0] != y)
                    continue;
                if (c->type == LAYER_ROCM_FUSED_LINEAR) {
                    auto cp = ParamOf<RocmFusedLinearParam>(c);
                    auto cr = ResOf<RocmFusedLinearResource>(c->name);
                    if (cr && !cp->ln_fold && cp->num_output % 8 == 0 && std::count(c->inputs.begin(), c->inputs.end(), y) == 1)
                        owner = ci, C = cr->weight_nk.GetBufferDims()[1];
                    ++owners;
                } else if (c->type == LAYER_ROCM_FUSED_ATTENTION) {
                    auto cp = ParamOf<RocmFusedAttentionParam>(c);
                    if (!cp->quant && !cp->ln_fold && cp->seq_len >= 0 && cp->seq_len % 8 == 0 &&
                        std::count(c->inputs.begin(), c->inputs.end(), y) == 1)
                        owner = ci, C = cp->heads * cp->head_dim;
                    ++owners;
                }
            }
            if (owners != 1 || owner < li || C <= 0 || C % 128 != 0)
                continue;
            RawBuffer *gamma = constant(ln->inputs[1], C), *beta = constant(ln->inputs[2], C);
            bool others = IsModelOutput(y), ordered = true;  // a model output is written like any other reader's copy
            for (int ci : cit->second)
                if (ci != owner) {
                    others = true;
                    ordered &= ci > owner;
                }
            if (!gamma || !beta || !ordered)
                continue;
            auto c = L[owner];
            auto cr = ResOf<RocmFusedLinearResource>(c->name);
            c->inputs[0] = t;
            cr->ln_gamma = *gamma;
            cr->ln_beta  = *beta;
            if (c->type == LAYER_ROCM_FUSED_LINEAR) {
                auto cp     = ParamOf<RocmFusedLinearParam>(c);
                cp->ln_fold = 1;
                cp->ln_y    = others ? 1 : 0;
                cp->ln_eps  = lp->eps;
            } else {
                auto cp     = ParamOf<RocmFusedAttentionParam>(c);
                cp->ln_fold = 1;
                cp->ln_y    = others ? 1 : 0;
                cp->ln_eps  = lp->eps;
            }
            if (others)
                c->outputs.push_back(y);
            L[li] = nullptr;
        }
        Compact();
    }

    // A folding layer (above) that still writes y = LayerNorm(t) because ONE other layer reads it, and that layer is a
    // RocmFusedLinear taking y as its residual operand (the block's residual Add): the folding layer hands over the
    // rows' {rstd, mean} instead (8 bytes per row, context side buffer named after y) and the residual reader takes t
    // and rebuilds y's values in its epilogue.  y is then neither written nor read: one tensor write and one tensor
    // read less per LayerNorm, same arithmetic per value.
    void HandOverRowStatistics() {
        auto &L = structure_->layers;
        for (int li = 0; li < (int)L.size(); ++li) {
            auto p = L[li];
            if (!p || (p->type != LAYER_ROCM_FUSED_LINEAR && p->type != LAYER_ROCM_FUSED_ATTENTION) || p->outputs.size() != 2)
                continue;
            auto pl = ParamOf<RocmFusedLinearParam>(p);
            auto pa = ParamOf<RocmFusedAttentionParam>(p);
            if (!(pl ? pl->ln_fold && pl->ln_y : pa && pa->ln_fold && pa->ln_y && !pa->out_quant))
                continue;
            auto pr = ResOf<RocmFusedLinearResource>(p->name);
            const std::string t = p->inputs[0], y = p->outputs[1];
            GraphIndex g(L);
            int ri = g.sole_consumer(y);
            if (!pr || ri <= li || IsModelOutput(y))
                continue;
            auto r  = L[ri];
            auto rp = r && r->type == LAYER_ROCM_FUSED_LINEAR ? ParamOf<RocmFusedLinearParam>(r) : nullptr;
            auto rr = rp ? ResOf<RocmFusedLinearResource>(r->name) : nullptr;
            if (!rp || !rr || !rp->has_residual || rp->ln_fold || rp->residual_ln || rp->axis >= 0 || r->inputs.size() != 2 ||
                r->inputs[1] != y || r->inputs[0] == y)
                continue;
            auto wd     = rr->weight_nk.GetBufferDims();
            const int C = pr->ln_gamma.GetDataCount();
            if (wd.size() != 2 || wd[0] != C || wd[1] % 64 != 0 || C % 8 != 0 || pr->ln_beta.GetDataCount() != C)
                continue;
            if (pl)
                pl->ln_y = 0, pl->ln_stats = 1, pl->ln_stats_key = y;
            else
                pa->ln_y = 0, pa->ln_stats = 1, pa->ln_stats_key = y;
            p->outputs.pop_back();
            r->inputs[1]        = t;
            rp->residual_ln     = 1;
            rp->residual_ln_key = y;
            rr->residual_gamma  = pr->ln_gamma;
            rr->residual_beta   = pr->ln_beta;
        }
    }

    // A folding layer reads t and needs every row's mean and variance.  When t is written by a RocmFusedLinear of the
    // residual_ln kind (above) whose rows are the normalised rows, that layer's GEMM leaves the rows' sums and sums of
    // squares per tile column next to t, and the folding GEMM adds them up while its first tiles are on their way,
    // instead of accumulating them from its A fragments in the main loop.
    void HandOverRowSums() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (auto &f : L) {
            if (!f || (f->type != LAYER_ROCM_FUSED_LINEAR && f->type != LAYER_ROCM_FUSED_ATTENTION))
                continue;
            auto fl = ParamOf<RocmFusedLinearParam>(f);
            auto fa = ParamOf<RocmFusedAttentionParam>(f);
            auto fr = ResOf<RocmFusedLinearResource>(f->name);
            if (!(fl ? fl->ln_fold : fa && fa->ln_fold) || !fr)
                continue;
            const std::string t = f->inputs[0];
            int gi = g.producer_of(t);
            auto w = gi >= 0 ? L[gi] : nullptr;
            auto wp = w && w->type == LAYER_ROCM_FUSED_LINEAR ? ParamOf<RocmFusedLinearParam>(w) : nullptr;
            const int C = fr->ln_gamma.GetDataCount();
            if (!wp || !wp->residual_ln || wp->num_output != C || C > 64 * TNN_ROCM_MAX_ROW_SUM_BLOCKS || !wp->row_sums_key.empty())
                continue;
            wp->row_sums_key = t;
            (fl ? fl->ln_sums_key : fa->ln_sums_key) = t;
        }
    }

    NetStructure *structure_ = nullptr;
    NetResource *resource_   = nullptr;
    bool half_               = true;
};

// ---- quantised nets -----------------------------------------------------------------------------------------------
// Quantised nets: insert float<->int8 Reformat layers wherever a quantised layer meets a float one.  The engine's own
// pass for this (source/tnn/optimizer/net_optimizer_insert_int8_reformat.cc:41-45, 66-216) serves ARM, NAIVE and X86
// only; this is the same rewrite for DEVICE_ROCM, at the same priority, so that the device needs no change there.
class RocmInsertInt8Reformat : public optimizer::NetOptimizer {
public:
    std::string Strategy() override { return "net_optimizer_rocm_insert_int8_reformat"; }
    bool IsSupported(const NetworkConfig &c) override {
        // the float side of every Reformat carries the network's float type, as the blobs around it do
        float_type_ = c.precision == PRECISION_HIGH ? DATA_TYPE_FLOAT
                                                    : (c.precision == PRECISION_LOW ? DATA_TYPE_BFP16 : DATA_TYPE_HALF);
        return c.device_type == DEVICE_ROCM;
    }
    Status Optimize(NetStructure *s, NetResource *res) override {
        RETURN_ON_NEQ(RocmCheckModel(s, res), TNN_OK);
        std::vector<std::shared_ptr<LayerInfo>> layers = s->layers;
        bool any_q  = false;
        for (auto &l : layers)
            any_q |= l->param->quantized;
        if (!any_q || layers.size() <= 1)
            return TNN_OK;
        std::vector<std::shared_ptr<LayerInfo>> out;
        const int count = (int)layers.size();
        // the Reformat layer behind `producer` (a layer, or a stand-in for a model input) for the blobs in `need`: readers
        // after position `index` whose kind differs from the producer's are redirected to its outputs
        // (net_optimizer_insert_int8_reformat.cc:183-216, AdjustLayer)
        auto insert_reformat = [&](const std::string &name, bool producer_quantized, const std::vector<std::string> &need,
                                   int index, std::shared_ptr<LayerInfo> *made) -> Status {
            auto nl      = std::make_shared<LayerInfo>();
            nl->type     = LAYER_REFORMAT;
            nl->type_str = "Reformat";
            nl->name     = name;
            auto p       = std::make_shared<ReformatLayerParam>();
            p->LayerParam::type = nl->type_str;  // ReformatLayerParam::type (quant direction) shadows the base field
            p->name      = nl->name;
            p->src_type  = producer_quantized ? DATA_TYPE_INT8 : float_type_;
            p->dst_type  = producer_quantized ? float_type_ : DATA_TYPE_INT8;
            nl->param    = p;
            nl->inputs   = need;
            for (auto &o : need) {
                std::string no = o + "_int8_reformat";
                nl->outputs.push_back(no);
                s->blobs.insert(no);
                for (int j = index + 1; j < count; ++j)
                    for (auto &in : layers[j]->inputs)
                        if (in == o && layers[j]->param->quantized != producer_quantized)
                            in = no;
                if (!producer_quantized) {
                    auto it = res->resource_map.find(o + "_scale_data_");
                    if (it == res->resource_map.end())
                        return Status(TNNERR_NULL_PARAM, "can not get blob scale " + o + "_scale_data_");
                    res->resource_map[no + "_scale_data_"] = it->second;
                }
            }
            *made = nl;
            return TNN_OK;
        };
        // A model input read by quantised and by float layers alike gets its Reformat at the head of the graph
        // (net_optimizer_insert_int8_reformat.cc:84-131); the input blob keeps the type the model declares for it.
        for (const auto &kv : s->inputs_shape_map) {
            const std::string &model_input = kv.first;
            int need_int8 = 0, need_float = 0;
            for (auto &l : layers)
                for (auto &in : l->inputs)
                    if (in == model_input) {
                        (l->param->quantized ? need_int8 : need_float)++;
                        break;
                    }
            if (need_int8 == 0 || need_float == 0)
                continue;
            auto ti = s->input_data_type_map.find(model_input);
            const DataType in_type = ti == s->input_data_type_map.end() ? DATA_TYPE_FLOAT : ti->second;
            if (in_type != DATA_TYPE_FLOAT && in_type != DATA_TYPE_INT8)
                return Status(TNNERR_UNSUPPORT_NET, "RocmInsertInt8Reformat: model input " + model_input +
                                                        " feeds quantised and float layers but is neither float nor int8");
            std::shared_ptr<LayerInfo> nl;
            RETURN_ON_NEQ(insert_reformat(model_input + "_int8_reformat__from_model_input__", in_type == DATA_TYPE_INT8,
                                          {model_input}, -1, &nl),
                          TNN_OK);
            out.push_back(nl);
        }
        for (int i = 0; i < count; ++i) {
            auto cur = layers[i];
            out.push_back(cur);
            if (cur->type == LAYER_REFORMAT)
                continue;
            std::vector<std::string> need;
            for (auto &o : cur->outputs) {
                bool n = false;
                for (int j = i + 1; j < count; ++j) {
                    if (layers[j]->type == LAYER_REFORMAT)
                        continue;
                    for (auto &in : layers[j]->inputs)
                        if (in == o && layers[j]->param->quantized != cur->param->quantized)
                            n = true;
                }
                if (n)
                    need.push_back(o);
            }
            if (need.empty())
                continue;
            std::shared_ptr<LayerInfo> nl;
            RETURN_ON_NEQ(insert_reformat(cur->name + "_int8_reformat", cur->param->quantized, need, i, &nl), TNN_OK);
            out.push_back(nl);
        }
        s->layers = out;
        return TNN_OK;
    }

private:
    DataType float_type_ = DATA_TYPE_FLOAT;
};


// Runs after the engine's own pass has made every float <-> int8 boundary an explicit Reformat layer
// (net_optimizer_insert_int8_reformat.cc:66-181).  A quantised encoder layer is then
//   Reformat(x) -> 3 x QuantizedInnerProduct -> 3 x Reformat -> head split, scores, softmax, P.V, head merge ->
//   Reformat -> QuantizedInnerProduct -> Reformat -> Add(residual) -> LayerNorm -> Reformat -> QuantizedInnerProduct
//   -> Reformat -> GELU -> Reformat -> QuantizedInnerProduct -> Reformat -> Add(residual) -> LayerNorm
// and this pass folds the Reformat layers into their neighbours, value for value:
//   * the three projections + their dequantising Reformats + the attention core  ==> RocmFusedAttention (quant)
//   * QuantizedInnerProduct -> Reformat(int8->float) [-> Add(residual)]            ==> RocmFusedLinearInt8
//   * Reformat(int8->float) -> GELU -> Reformat(float->int8)                       ==> RocmGeluInt8
//   * LayerNorm -> Reformat(float->int8)                                           ==> LayerNorm with a second, int8 output
// Each fused kernel forms the same int8 values as the chain it replaces (requantisation and quantisation are the
// reference's float2int8 steps); float intermediates that the chain would have rounded to the blob type (fp16 nets)
// stay in fp32 inside the fused kernel.
class RocmInt8FusionPass : public optimizer::NetOptimizer {
public:
    std::string Strategy() override { return "net_optimizer_rocm_fuse_int8"; }
    bool IsSupported(const NetworkConfig &c) override {
        half_ = c.precision != PRECISION_HIGH;
        const char *e = getenv("TNN_ROCM_FUSE_INT8");  // "0" keeps the explicit Reformat chain (used by the tests)
        return c.device_type == DEVICE_ROCM && !(e && atoi(e) == 0);
    }
    Status Optimize(NetStructure *s, NetResource *r) override {
        RETURN_ON_NEQ(RocmCheckModel(s, r), TNN_OK);
        structure_ = s;
        resource_  = r;
        bool any_q = false;
        for (auto &l : s->layers)
            any_q |= l->param->quantized;
        if (!any_q)
            return TNN_OK;
        if (half_)
            FuseAttention();
        FoldGelu();
        FoldGeluIntoProjection();
        FoldDequant();
        FoldLayerNormQuant();
        FoldAttentionQuant();
        return TNN_OK;
    }

private:
    bool IsModelOutput(const std::string &b) const { return structure_->outputs.count(b) > 0; }
    void Compact() {
        auto &L = structure_->layers;
        L.erase(std::remove(L.begin(), L.end(), nullptr), L.end());
    }
    template <typename T> T *ParamOf(const std::shared_ptr<LayerInfo> &l) { return dynamic_cast<T *>(l->param.get()); }
    template <typename T> T *ResOf(const std::string &name) {
        auto it = resource_->resource_map.find(name);
        return it == resource_->resource_map.end() ? nullptr : dynamic_cast<T *>(it->second.get());
    }
    bool BlobScale(const std::string &blob, float *scale) {
        auto r = ResOf<IntScaleResource>(blob + "_scale_data_");
        if (!r || r->scale_handle.GetDataCount() != 1 || r->scale_handle.GetDataType() != DATA_TYPE_FLOAT)
            return false;
        *scale = r->scale_handle.force_to<float *>()[0];
        return true;
    }
    // single-input, single-output Reformat in the given direction
    bool IsReformat(const std::shared_ptr<LayerInfo> &l, bool to_int8) {
        if (!l || l->type != LAYER_REFORMAT || l->inputs.size() != 1 || l->outputs.size() != 1)
            return false;
        auto p = ParamOf<ReformatLayerParam>(l);
        return p && (to_int8 ? (p->src_type != DATA_TYPE_INT8 && p->dst_type == DATA_TYPE_INT8)
                             : (p->src_type == DATA_TYPE_INT8 && p->dst_type != DATA_TYPE_INT8));
    }
    bool IsQuantFc(const std::shared_ptr<LayerInfo> &l) {
        if (!l || l->type != LAYER_INNER_PRODUCT || !l->param->quantized || l->inputs.size() != 1)
            return false;
        auto ip = ParamOf<InnerProductLayerParam>(l);
        auto ir = ResOf<InnerProductLayerResource>(l->name);
        return ip && ir && ip->axis == 1 && ir->weight_handle.GetDataType() == DATA_TYPE_INT8 && ip->num_output > 0 &&
               ir->weight_handle.GetDataCount() % ip->num_output == 0 &&
               (ir->scale_handle.GetDataCount() == ip->num_output || ir->scale_handle.GetDataCount() == 1);
    }

    // `blob` <- Permute(order) <- Reshape(head split) <- Reformat(int8->float) <- QuantizedInnerProduct
    int QuantHeadSplitSource(const GraphIndex &g, const std::string &blob, const std::vector<int> &order4,
                             const std::vector<int> &order3, std::vector<int> *chain, DimsVector *split_shape) {
        auto &L = structure_->layers;
        int pi  = g.producer_of(blob);
        if (pi < 0 || !L[pi] || L[pi]->type != LAYER_PERMUTE || g.sole_consumer(blob) < 0 || IsModelOutput(blob))
            return -1;
        auto pp = ParamOf<PermuteLayerParam>(L[pi]);
        if (!pp || (pp->orders != order4 && pp->orders != order3))
            return -1;
        const std::string &rb = L[pi]->inputs[0];
        int ri                = g.producer_of(rb);
        if (ri < 0 || !L[ri] || L[ri]->type != LAYER_RESHAPE || g.sole_consumer(rb) != pi || IsModelOutput(rb))
            return -1;
        auto rp = ParamOf<ReshapeLayerParam>(L[ri]);
        if (!rp || rp->axis != 0 || rp->shape.size() != pp->orders.size() || L[ri]->inputs.size() != 1)
            return -1;
        const std::string &fb = L[ri]->inputs[0];
        int fi                = g.producer_of(fb);
        if (fi < 0 || !IsReformat(L[fi], false) || g.sole_consumer(fb) != ri || IsModelOutput(fb))
            return -1;
        const std::string &qb = L[fi]->inputs[0];
        int li                = g.producer_of(qb);
        if (li < 0 || !IsQuantFc(L[li]) || g.sole_consumer(qb) != fi || IsModelOutput(qb))
            return -1;
        chain->push_back(pi);
        chain->push_back(ri);
        chain->push_back(fi);
        chain->push_back(li);
        *split_shape = rp->shape;
        return li;
    }

    void FuseAttention() {
        auto &L = structure_->layers;
        bool changed = true;
        while (changed) {
            changed = false;
            GraphIndex g(L);
            for (int si = 0; si < (int)L.size() && !changed; ++si) {
                auto sm = L[si];
                if (!sm || sm->type != LAYER_SOFTMAX)
                    continue;
                AttentionCore m;
                AttentionMatcher matcher(structure_, resource_,
                                         [this](const GraphIndex &gi, const std::string &blob, const std::vector<int> &o4,
                                                const std::vector<int> &o3, std::vector<int> *chain, DimsVector *shape) {
                                             return QuantHeadSplitSource(gi, blob, o4, o3, chain, shape);
                                         });
                if (!matcher.Match(g, si, &m))
                    continue;
                const std::vector<int> &chain = m.chain;
                const std::string &mask = m.mask;
                const float scale = m.scale;
                const int lq = m.lq, lk = m.lk, lv = m.lv, rs = m.rs;
                const DimsVector &shape_q = m.split_shape;
                // the three projections read the same int8 blob and have the same shape
                if (L[lq]->inputs[0] != L[lk]->inputs[0] || L[lq]->inputs[0] != L[lv]->inputs[0])
                    continue;
                InnerProductLayerResource *src[3] = {ResOf<InnerProductLayerResource>(L[lq]->name),
                                                     ResOf<InnerProductLayerResource>(L[lk]->name),
                                                     ResOf<InnerProductLayerResource>(L[lv]->name)};
                int H = ParamOf<InnerProductLayerParam>(L[lq])->num_output;
                if (ParamOf<InnerProductLayerParam>(L[lk])->num_output != H || ParamOf<InnerProductLayerParam>(L[lv])->num_output != H)
                    continue;
                int K = src[0]->weight_handle.GetDataCount() / H;
                if (src[1]->weight_handle.GetDataCount() != H * K || src[2]->weight_handle.GetDataCount() != H * K)
                    continue;
                int heads = shape_q[shape_q.size() - 2], head_dim = shape_q.back(), seq = shape_q[shape_q.size() - 3];
                if (heads * head_dim != H || head_dim != 64 || seq <= 0 || seq % 8 != 0 || K % 64 != 0)
                    continue;
                float out_scale[3];
                if (!BlobScale(L[lq]->outputs[0], &out_scale[0]) || !BlobScale(L[lk]->outputs[0], &out_scale[1]) ||
                    !BlobScale(L[lv]->outputs[0], &out_scale[2]))
                    continue;
                int first = *std::min_element(chain.begin(), chain.end());
                auto fl      = std::make_shared<LayerInfo>();
                fl->type     = LAYER_ROCM_FUSED_ATTENTION;
                fl->type_str = "RocmFusedAttention";
                fl->name     = sm->name + "_fused_attention_int8";
                fl->inputs   = {L[lq]->inputs[0]};
                if (!mask.empty())
                    fl->inputs.push_back(mask);
                fl->outputs  = {L[rs]->outputs[0]};
                auto fp      = std::make_shared<RocmFusedAttentionParam>();
                fp->type     = fl->type_str;
                fp->name     = fl->name;
                fp->heads    = heads;
                fp->head_dim = head_dim;
                fp->scale    = scale;
                fp->has_mask = mask.empty() ? 0 : 1;
                fp->split_rank  = (int)shape_q.size();
                fp->merge_shape = ParamOf<ReshapeLayerParam>(L[rs])->shape;
                fp->seq_len  = seq;
                fp->quant    = 1;
                for (int t = 0; t < 3; ++t)
                    fp->qkv_out_scale[t] = out_scale[t];
                fl->param    = fp;
                auto fr      = std::make_shared<RocmFusedQkvInt8Resource>();
                fr->name     = fl->name;
                fr->weight   = RawBuffer(3 * H * K, {3 * H, K});
                fr->weight.SetDataType(DATA_TYPE_INT8);
                fr->bias     = RawBuffer(3 * H * 4, {3 * H});
                fr->bias.SetDataType(DATA_TYPE_INT32);
                fr->w_scale  = RawBuffer(3 * H * 4, {3 * H});
                memset(fr->bias.force_to<void *>(), 0, (size_t)3 * H * 4);
                for (int t = 0; t < 3; ++t) {
                    memcpy(fr->weight.force_to<int8_t *>() + (size_t)t * H * K, src[t]->weight_handle.force_to<int8_t *>(),
                           (size_t)H * K);
                    if (src[t]->bias_handle.GetDataCount() == H)
                        memcpy(fr->bias.force_to<int32_t *>() + (size_t)t * H, src[t]->bias_handle.force_to<int32_t *>(),
                               (size_t)H * 4);
                    const float *ws = src[t]->scale_handle.force_to<float *>();
                    int n_ws        = src[t]->scale_handle.GetDataCount();
                    for (int i = 0; i < H; ++i)
                        fr->w_scale.force_to<float *>()[(size_t)t * H + i] = ws[n_ws == 1 ? 0 : i];
                }
                resource_->resource_map[fl->name] = fr;
                for (int idx : chain)
                    L[idx] = nullptr;
                L[first] = fl;
                changed  = true;
            }
            Compact();
        }
    }

    // int8 h -> Reformat(int8->float) -> GELU -> Reformat(float->int8) -> int8 g    ==>   RocmGeluInt8(h) -> g
    void FoldGelu() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            if (!IsReformat(L[i], false) || IsModelOutput(L[i]->outputs[0]))
                continue;
            int gi = g.sole_consumer(L[i]->outputs[0]);
            if (gi < 0 || !L[gi] || L[gi]->type != LAYER_GELU || IsModelOutput(L[gi]->outputs[0]))
                continue;
            int ri = g.sole_consumer(L[gi]->outputs[0]);
            if (ri < 0 || !IsReformat(L[ri], true))
                continue;
            auto nl      = std::make_shared<LayerInfo>();
            nl->type     = LAYER_ROCM_GELU_INT8;
            nl->type_str = "RocmGeluInt8";
            nl->name     = L[gi]->name + "_int8";
            nl->inputs   = {L[i]->inputs[0]};
            nl->outputs  = {L[ri]->outputs[0]};
            auto p       = std::make_shared<LayerParam>();
            p->type      = nl->type_str;
            p->name      = nl->name;
            p->quantized = true;
            nl->param    = p;
            L[i]  = nl;
            L[gi] = nullptr;
            L[ri] = nullptr;
        }
        Compact();
    }

    // QuantizedInnerProduct -> int8 h -> RocmGeluInt8 -> int8 g   ==>   RocmQuantLinearGelu -> g  (the GELU chain has 256
    // possible inputs: the projection applies it as a table in its epilogue).  TNN_ROCM_FOLD_GELU_LUT=0 keeps two launches.
    void FoldGeluIntoProjection() {
        const char *sw = getenv("TNN_ROCM_FOLD_GELU_LUT");
        if (sw && sw[0] == '0')
            return;
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            if (!IsQuantFc(L[i]) || IsModelOutput(L[i]->outputs[0]))
                continue;
            int gi = g.sole_consumer(L[i]->outputs[0]);
            float mid_scale;
            if (gi < 0 || !L[gi] || L[gi]->type != LAYER_ROCM_GELU_INT8 || !BlobScale(L[i]->outputs[0], &mid_scale))
                continue;
            auto ip = ParamOf<InnerProductLayerParam>(L[i]);
            auto np = std::make_shared<RocmQuantLinearGeluParam>();
            static_cast<InnerProductLayerParam &>(*np) = *ip;
            np->type      = "RocmQuantLinearGelu";
            np->quantized = true;
            np->mid_scale = mid_scale;
            auto nl       = std::make_shared<LayerInfo>(*L[i]);  // keeps the name: the resource is looked up by it
            nl->type      = LAYER_ROCM_QUANT_LINEAR_GELU;
            nl->type_str  = "RocmQuantLinearGelu";
            nl->param     = np;
            nl->outputs   = {L[gi]->outputs[0]};
            L[i]  = nl;
            L[gi] = nullptr;
        }
        Compact();
    }

    // QuantizedInnerProduct -> int8 y -> Reformat(int8->float) [-> Add(other)]   ==>   RocmFusedLinearInt8
    void FoldDequant() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            if (!IsQuantFc(L[i]) || IsModelOutput(L[i]->outputs[0]))
                continue;
            int ri = g.sole_consumer(L[i]->outputs[0]);
            if (ri < 0 || !IsReformat(L[ri], false))
                continue;
            float out_scale;
            if (!BlobScale(L[i]->outputs[0], &out_scale))
                continue;
            auto ip      = ParamOf<InnerProductLayerParam>(L[i]);
            auto np      = std::make_shared<RocmFusedLinearInt8Param>();
            static_cast<InnerProductLayerParam &>(*np) = *ip;
            np->type      = "RocmFusedLinearInt8";
            np->quantized = true;
            np->out_scale = out_scale;
            auto nl       = std::make_shared<LayerInfo>(*L[i]);  // keeps the name: the resource is looked up by it
            nl->type      = LAYER_ROCM_FUSED_LINEAR_INT8;
            nl->type_str  = "RocmFusedLinearInt8";
            nl->param     = np;
            nl->outputs   = {L[ri]->outputs[0]};
            // residual: the dequantised value's only reader is a float two-input Add whose other operand exists already
            const std::string &y = L[ri]->outputs[0];
            int ai               = g.sole_consumer(y);
            if (ai > ri && L[ai] && L[ai]->type == LAYER_ADD && L[ai]->inputs.size() == 2 && !L[ai]->param->quantized &&
                !ResOf<EltwiseLayerResource>(L[ai]->name) && !IsModelOutput(y)) {
                const std::string &other = L[ai]->inputs[0] == y ? L[ai]->inputs[1] : L[ai]->inputs[0];
                int po = g.producer_of(other);
                bool available = other != y && (po >= 0 ? po < i : structure_->inputs_shape_map.count(other) > 0);
                if (available) {
                    np->has_residual = 1;
                    nl->inputs.push_back(other);
                    nl->outputs = {L[ai]->outputs[0]};
                    L[ai]       = nullptr;
                }
            }
            L[i]  = nl;
            L[ri] = nullptr;
        }
        Compact();
    }

    // LayerNorm -> float x -> Reformat(float->int8) -> int8 xq   ==>   LayerNorm with outputs {x, xq}
    void FoldLayerNormQuant() {
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            if (!L[i] || L[i]->type != LAYER_LAYER_NORM || L[i]->outputs.size() != 1)
                continue;
            auto it = g.consumers.find(L[i]->outputs[0]);
            if (it == g.consumers.end())
                continue;
            for (int ri : it->second) {
                if (ri > i && IsReformat(L[ri], true)) {
                    // a layer type of its own: the engine's LayerNorm layer class infers shape and type of one output
                    L[i]->outputs.push_back(L[ri]->outputs[0]);
                    L[i]->type     = LAYER_ROCM_LAYER_NORM_QUANT;
                    L[i]->type_str = "RocmLayerNormQuant";
                    L[ri] = nullptr;
                    break;
                }
            }
        }
        Compact();
    }

    // RocmFusedAttention -> Reformat(float -> int8): the attention kernel writes the quantised context as a second
    // output in the same launch (the float one stays for any other reader)
    void FoldAttentionQuant() {
        const char *sw = getenv("TNN_ROCM_FOLD_ATTN_Q8");
        if (sw && sw[0] == '0')
            return;
        auto &L = structure_->layers;
        GraphIndex g(L);
        for (int i = 0; i < (int)L.size(); ++i) {
            if (!L[i] || L[i]->type != LAYER_ROCM_FUSED_ATTENTION || L[i]->outputs.size() != 1)
                continue;
            auto ap = ParamOf<RocmFusedAttentionParam>(L[i]);
            if (!ap || ap->seq_len <= 0 || ap->seq_len % 8 != 0)  // the V^T form of the kernel carries the second output
                continue;
            auto it = g.consumers.find(L[i]->outputs[0]);
            if (it == g.consumers.end())
                continue;
            for (int ri : it->second) {
                if (ri > i && IsReformat(L[ri], true)) {
                    L[i]->outputs.push_back(L[ri]->outputs[0]);
                    ap->out_quant = 1;
                    L[ri]         = nullptr;
                    break;
                }
            }
        }
        Compact();
    }

    NetStructure *structure_ = nullptr;
    NetResource *resource_   = nullptr;
    bool half_               = true;
};

// optimizer/net_optimizer_manager.cc:33-48 runs the passes sorted by (priority, strategy name): the float rewrite runs
// with the engine's own fusions (P1); the Reformat insertion at the priority of the engine's own (P2); the int8 rewrite
// needs the Reformat layers and runs last (PLAST; the engine's only other pass there, the layout Reformat insertion,
// sorts in front of it by name and finds one layout everywhere on this device)
optimizer::NetOptimizerRegister<RocmFusionPass> g_net_optimizer_rocm_fuse_encoder(optimizer::P1);
optimizer::NetOptimizerRegister<RocmInsertInt8Reformat> g_net_optimizer_rocm_insert_int8_reformat(optimizer::P2);
optimizer::NetOptimizerRegister<RocmInt8FusionPass> g_net_optimizer_rocm_fuse_int8(optimizer::PLAST);

}  // namespace

// ---- LayerNorm folded into a projection: weight preparation ---------------------------------------------------
// value of f after rounding to the activation type (round to nearest even, as the device conversion does)
static float RoundToActivationType(float f, DataType dt) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = x & 0x80000000u, a = x & 0x7fffffffu;
    if (a >= 0x7f800000u)
        return f;
    if (dt == DATA_TYPE_BFP16) {
        a = (a + 0x7fffu + ((a >> 16) & 1u)) & 0xffff0000u;
    } else if (a < 0x38800000u) {  // below 2^-14: a multiple of the fp16 subnormal step 2^-24
        float af;
        memcpy(&af, &a, 4);
        af = (af + 0.5f) - 0.5f;  // the sum has an ulp of 2^-24: rounds af to that grid, ties to even
        memcpy(&a, &af, 4);
    } else {
        a = (a + 0xfffu + ((a >> 13) & 1u)) & 0xffffe000u;
        if (a >= 0x47800000u)  // 65520 and above round to infinity
            a = 0x7f800000u;
    }
    x = sign | a;
    memcpy(&f, &x, 4);
    return f;
}

// y W^T + b with y = (t - mean) * rstd * gamma + beta  ==  rstd * (t W'^T - mean * colsum) + b'
//   W'[n,k] = gamma[k] W[n,k] (as the device will hold it, i.e. rounded to dt),  colsum[n] = sum_k W'[n,k],
//   b'[n] = b[n] + sum_k beta[k] W[n,k]
static void FoldLayerNormIntoWeights(const float *w, const float *bias, const float *gamma, const float *beta, int N, int K,
                                     DataType dt, std::vector<float> *w_folded, std::vector<float> *colsum,
                                     std::vector<float> *bias_folded) {
    w_folded->resize((size_t)N * K);
    colsum->resize(N);
    bias_folded->resize(N);
    for (int n = 0; n < N; ++n) {
        double cs = 0.0, bs = bias ? (double)bias[n] : 0.0;
        for (int k = 0; k < K; ++k) {
            float wf = RoundToActivationType(w[(size_t)n * K + k] * gamma[k], dt);
            (*w_folded)[(size_t)n * K + k] = wf;
            cs += (double)wf;
            bs += (double)beta[k] * (double)w[(size_t)n * K + k];
        }
        (*colsum)[n]      = (float)cs;
        (*bias_folded)[n] = (float)bs;
    }
}

// the side buffer a residual_ln layer leaves its output's row sums in: room for the most tile columns a launch may have
static size_t RowSumsBytes(int rows) { return (size_t)TNN_ROCM_MAX_ROW_SUM_BLOCKS * (size_t)rows * 2 * sizeof(float); }
// what a folding layer finds there: the buffer and the block count of the launch that wrote it (0 blocks, or no key:
// nothing was handed over and the GEMM takes the statistics itself)
static Status RowSumsOf(RocmContext *ctx, const std::string &key, int rows, void **sums, int *blocks) {
    *sums   = nullptr;
    *blocks = 0;
    if (key.empty())
        return TNN_OK;
    *blocks = ctx->SideBufferTag(key);
    if (*blocks > 0)
        return ctx->SideBuffer(key, RowSumsBytes(rows), sums);
    return TNN_OK;
}

// ---- RocmFusedLinear ------------------------------------------------------------------------------------------
// y[rows,N] = act(x[rows,K] W^T + b) (+ residual): the arithmetic of MatMul+Add (cpu_mat_mul_layer_acc.cc:64-117,
// compute_elewise.cc:37-65) or InnerProduct (naive_compute.cc:271-288), GELU (cpu_gelu_layer_acc.cc:42-45) and the
// residual Add, in one MFMA GEMM launch with the epilogue applied on the fp32 accumulators.
class RocmFusedLinearLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        if (weight_)
            return TNN_OK;
        auto res = dynamic_cast<RocmFusedLinearResource *>(resource_);
        auto p   = dynamic_cast<RocmFusedLinearParam *>(param_);
        CHECK_PARAM_NULL(res);
        CHECK_PARAM_NULL(p);
        auto wd = res->weight_nk.GetBufferDims();
        auto in = inputs[0]->GetBlobDesc().dims;
        int k_in = p->axis >= 0 ? DimsVectorUtils::Count(in, p->axis) : (in.empty() ? 0 : in.back());
        if (wd.size() != 2 || in.empty() || k_in != wd[1] || wd[0] != p->num_output)
            return Status(TNNERR_PARAM_ERR, "fused linear: weight [N,K] does not match the contracted input dimensions");
        if (p->has_residual) {
            if (inputs.size() != 2 || inputs[1]->GetBlobDesc().dims != outputs[0]->GetBlobDesc().dims ||
                inputs[1]->GetBlobDesc().data_type != outputs[0]->GetBlobDesc().data_type)
                return Status(TNNERR_PARAM_ERR, "fused linear: residual must have the output's shape and type");
        }
        DataType dt = inputs[0]->GetBlobDesc().data_type;
        if (p->residual_ln) {
            if ((dt != DATA_TYPE_HALF && dt != DATA_TYPE_BFP16) || p->ln_fold || !p->has_residual || wd[1] % 64 != 0 || wd[0] % 8 != 0 ||
                res->residual_gamma.GetDataCount() != wd[0] || res->residual_beta.GetDataCount() != wd[0])
                return Status(TNNERR_PARAM_ERR, "fused linear with a rebuilt LayerNorm residual: fp16/bf16 blobs, K a multiple "
                                                "of 64 and scale / shift of the output width are required");
            RETURN_ON_NEQ(UploadConverted(res->residual_gamma.force_to<void *>(), (size_t)wd[0], DATA_TYPE_FLOAT, DATA_TYPE_FLOAT,
                                          &res_gamma_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->residual_beta.force_to<void *>(), (size_t)wd[0], DATA_TYPE_FLOAT, DATA_TYPE_FLOAT,
                                          &res_beta_), TNN_OK);
        }
        if (p->ln_fold) {
            if ((dt != DATA_TYPE_HALF && dt != DATA_TYPE_BFP16) || outputs.size() != (p->ln_y ? 2u : 1u) || in.back() != wd[1] ||
                wd[1] % 128 != 0 || wd[0] % 8 != 0 || res->ln_gamma.GetDataCount() != wd[1] || res->ln_beta.GetDataCount() != wd[1])
                return Status(TNNERR_PARAM_ERR, "fused linear with a folded LayerNorm: fp16/bf16 blobs, the last axis (a "
                                                "multiple of 128) contracted, scale / shift of that width are required");
            std::vector<float> wf, cs, bf;
            FoldLayerNormIntoWeights(res->weight_nk.force_to<float *>(), p->has_bias ? res->bias.force_to<float *>() : nullptr,
                                     res->ln_gamma.force_to<float *>(), res->ln_beta.force_to<float *>(), wd[0], wd[1], dt, &wf,
                                     &cs, &bf);
            RETURN_ON_NEQ(UploadConverted(wf.data(), wf.size(), DATA_TYPE_FLOAT, dt, &weight_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(bf.data(), bf.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &bias_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(cs.data(), cs.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &colsum_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->ln_gamma.force_to<void *>(), (size_t)wd[1], DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &gamma_),
                          TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->ln_beta.force_to<void *>(), (size_t)wd[1], DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &beta_),
                          TNN_OK);
        } else {
            RETURN_ON_NEQ(UploadConverted(res->weight_nk.force_to<void *>(), (size_t)wd[0] * wd[1], DATA_TYPE_FLOAT, dt, &weight_),
                          TNN_OK);
            if (p->has_bias)
                RETURN_ON_NEQ(UploadConverted(res->bias.force_to<void *>(), (size_t)wd[0], DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &bias_),
                              TNN_OK);
        }
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto p  = dynamic_cast<RocmFusedLinearParam *>(param_);
        auto in = inputs[0]->GetBlobDesc().dims;
        int K = p->axis >= 0 ? DimsVectorUtils::Count(in, p->axis) : in.back();
        int N = p->num_output, rows = DimsVectorUtils::Count(in) / (K > 0 ? K : 1);
        int epi = (p->has_bias ? TNN_ROCM_EPI_BIAS : 0) | (p->gelu ? TNN_ROCM_EPI_GELU : 0) |
                  (p->has_residual ? TNN_ROCM_EPI_RESIDUAL : 0);
        if (p->ln_fold) {
            void *stats = nullptr, *sums = nullptr;
            int blocks = 0;
            if (p->ln_stats)
                RETURN_ON_NEQ(context_->SideBuffer(p->ln_stats_key, (size_t)rows * 2 * sizeof(float), &stats), TNN_OK);
            RETURN_ON_NEQ(RowSumsOf(context_, p->ln_sums_key, rows, &sums, &blocks), TNN_OK);
            ROCM_CALL(tnn_rocm_gemm_ln(Stream(), (int)inputs[0]->GetBlobDesc().data_type, Ptr(inputs[0]), weight_,
                                       (const float *)bias_, (const float *)colsum_, (const float *)gamma_, (const float *)beta_,
                                       p->ln_eps, Ptr(outputs[0]), p->ln_y ? Ptr(outputs[1]) : nullptr, (float *)stats,
                                       (const float *)sums, blocks, rows, N, K, epi & ~TNN_ROCM_EPI_BIAS,
                                       p->has_residual ? Ptr(In(inputs[1])) : nullptr));
            return TNN_OK;
        }
        if (p->residual_ln) {
            void *stats = nullptr;
            RETURN_ON_NEQ(context_->SideBuffer(p->residual_ln_key, (size_t)rows * 2 * sizeof(float), &stats), TNN_OK);
            void *sums = nullptr;
            int blocks = 0;
            if (!p->row_sums_key.empty())
                RETURN_ON_NEQ(context_->SideBuffer(p->row_sums_key, RowSumsBytes(rows), &sums), TNN_OK);
            ROCM_CALL(tnn_rocm_gemm_residual_ln(Stream(), (int)inputs[0]->GetBlobDesc().data_type, Ptr(inputs[0]), weight_,
                                                (const float *)bias_, Ptr(outputs[0]), Ptr(In(inputs[1])), (const float *)stats,
                                                (const float *)res_gamma_, (const float *)res_beta_, rows, N, K,
                                                epi & ~TNN_ROCM_EPI_RESIDUAL, (float *)sums, sums ? &blocks : nullptr));
            if (sums)
                context_->SideBufferTag(p->row_sums_key) = blocks;
            return TNN_OK;
        }
        ROCM_CALL(tnn_rocm_gemm(Stream(), (int)inputs[0]->GetBlobDesc().data_type, 1, Ptr(inputs[0]), weight_, Ptr(outputs[0]),
                                rows, N, K, K, K, N, 1, 1, 1, epi, (const float *)bias_,
                                p->has_residual ? Ptr(In(inputs[1])) : nullptr, N));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr, *bias_ = nullptr, *colsum_ = nullptr, *gamma_ = nullptr, *beta_ = nullptr, *res_gamma_ = nullptr,
         *res_beta_ = nullptr;
};
REGISTER_ROCM_ACC(RocmFusedLinearLayerAcc, LAYER_ROCM_FUSED_LINEAR);

// ---- RocmFusedAttention -----------------------------------------------------------------------------------------
// x [B,S,H] (or [T,H]) -> packed QKV = x Wqkv^T + bqkv in the context workspace -> flash-style attention kernel
// reading Q/K/V straight out of the packed buffer (no Reshape/Permute copies) -> ctx [B,S,H].
// The additive mask blob (broadcastable to [B,1,1,S]) is brought to fp32 [B,S] once per forward; from it the
// per-sequence valid length is derived on the device so whole key tiles of padding are skipped.
class RocmFusedAttentionLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto res  = dynamic_cast<RocmFusedLinearResource *>(resource_);
        auto res8 = dynamic_cast<RocmFusedQkvInt8Resource *>(resource_);
        auto p    = dynamic_cast<RocmFusedAttentionParam *>(param_);
        CHECK_PARAM_NULL(p);
        if (p->quant ? !res8 : !res)
            return Status(TNNERR_NULL_PARAM, "fused attention: resource is nil");
        auto in = inputs[0]->GetBlobDesc().dims;
        H_      = p->heads * p->head_dim;
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        if (dt != DATA_TYPE_HALF && dt != DATA_TYPE_BFP16)
            return Status(TNNERR_LAYER_ERR, "fused attention runs in fp16/bf16 only");
        if (p->quant) {
            auto wd = res8->weight.GetBufferDims();
            if (in.empty() || wd.size() != 2 || wd[0] != 3 * H_ || in.back() != wd[1] ||
                inputs[0]->GetBlobDesc().data_type != DATA_TYPE_INT8)
                return Status(TNNERR_PARAM_ERR, "fused int8 attention: input / weight shape mismatch");
            K_ = wd[1];
        } else {
            if (in.empty() || in.back() != H_ || res->weight_nk.GetBufferDims() != DimsVector({3 * H_, H_}))
                return Status(TNNERR_PARAM_ERR, "fused attention: hidden size mismatch");
            K_ = H_;
        }
        T_   = DimsVectorUtils::Count(in) / K_;
        seq_ = p->seq_len > 0 ? p->seq_len : (in.size() >= 3 ? in[in.size() - 2] : T_);
        if (seq_ <= 0 || T_ % seq_ != 0)
            return Status(TNNERR_PARAM_ERR, "fused attention: token count is not a multiple of the sequence length");
        B_ = T_ / seq_;
        if (p->has_mask) {
            // one additive value per key: [B,1,1,S], or one row [1,1,1,S] for every sequence
            const int count = inputs.size() < 2 ? -1 : DimsVectorUtils::Count(In(inputs[1])->GetBlobDesc().dims);
            if (count != B_ * seq_ && count != seq_)
                return Status(TNNERR_PARAM_ERR, "fused attention: mask must hold B*S (or S) additive values");
            mask_one_row_ = count == seq_ && B_ > 1;
        }
        if (!weight_ && p->quant) {
            // requantisation factor w_scale / o_scale of each projection as one fp32 division on the host, 0 when
            // o_scale < FLT_MIN (x86_inner_product_layer_acc.cc:197-222); dequantisation = the projection's blob scale
            const int N = 3 * H_;
            std::vector<float> scale(N), dequant(N);
            const float *ws = res8->w_scale.force_to<float *>();
            for (int i = 0; i < N; ++i) {
                float os   = p->qkv_out_scale[i / H_];
                scale[i]   = os >= FLT_MIN ? ws[i] / os : 0.0f;
                dequant[i] = os;
            }
            RETURN_ON_NEQ(UploadConverted(res8->weight.force_to<void *>(), (size_t)N * K_, DATA_TYPE_INT8, DATA_TYPE_INT8, &weight_),
                          TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res8->bias.force_to<void *>(), (size_t)N, DATA_TYPE_INT32, DATA_TYPE_INT32, &bias_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(scale.data(), (size_t)N, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &scale_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(dequant.data(), (size_t)N, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &dequant_), TNN_OK);
        }
        if (!weight_ && p->ln_fold) {
            if (p->quant || H_ % 128 != 0 || outputs.size() != 1u + (p->ln_y ? 1u : 0u) + (p->out_quant ? 1u : 0u) ||
                res->ln_gamma.GetDataCount() != H_ || res->ln_beta.GetDataCount() != H_)
                return Status(TNNERR_PARAM_ERR, "fused attention with a folded LayerNorm: a hidden size that is a multiple "
                                                "of 128 and scale / shift of that width are required");
            std::vector<float> wf, cs, bf;
            FoldLayerNormIntoWeights(res->weight_nk.force_to<float *>(), res->bias.force_to<float *>(),
                                     res->ln_gamma.force_to<float *>(), res->ln_beta.force_to<float *>(), 3 * H_, H_, dt, &wf, &cs,
                                     &bf);
            RETURN_ON_NEQ(UploadConverted(wf.data(), wf.size(), DATA_TYPE_FLOAT, dt, &weight_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(bf.data(), bf.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &bias_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(cs.data(), cs.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &colsum_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->ln_gamma.force_to<void *>(), (size_t)H_, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &gamma_), TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->ln_beta.force_to<void *>(), (size_t)H_, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &beta_), TNN_OK);
        }
        if (!weight_) {
            RETURN_ON_NEQ(UploadConverted(res->weight_nk.force_to<void *>(), (size_t)3 * H_ * H_, DATA_TYPE_FLOAT, dt, &weight_),
                          TNN_OK);
            RETURN_ON_NEQ(UploadConverted(res->bias.force_to<void *>(), (size_t)3 * H_, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &bias_),
                          TNN_OK);
        }
        return TNN_OK;
    }

    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto p      = dynamic_cast<RocmFusedAttentionParam *>(param_);
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        size_t es   = (size_t)DataTypeUtils::GetBytesSize(dt);
        void *qkv   = nullptr;
        RETURN_ON_NEQ(context_->Workspace((size_t)T_ * 3 * H_ * es, &qkv), TNN_OK);
        void *stats = nullptr;  // the folded LayerNorm's {rstd, mean} per row, for the layer that rebuilds its output
        if (p->ln_fold && p->ln_stats)
            RETURN_ON_NEQ(context_->SideBuffer(p->ln_stats_key, (size_t)T_ * 2 * sizeof(float), &stats), TNN_OK);
        void *sums = nullptr;  // the rows' sums left by the layer that wrote the input, see HandOverRowSums
        int blocks = 0;
        if (p->ln_fold)
            RETURN_ON_NEQ(RowSumsOf(context_, p->ln_sums_key, T_, &sums, &blocks), TNN_OK);
        const float *mask = nullptr;
        const int32_t *kv = nullptr;
        if (p->has_mask) {
            Blob *mb = In(inputs[1]);
            RETURN_ON_NEQ(context_->AttentionMask(Ptr(mb), (int)mb->GetBlobDesc().data_type, B_, seq_, mask_one_row_, &mask, &kv),
                          TNN_OK);
        }
        const char *base = (const char *)qkv;
        const long d     = p->head_dim;
        // V^T leaves the projection with its keys in the order the attention kernel's accumulators hold them (no
        // register exchange in front of the second MFMA) whenever whole groups of 16 keys exist
        const int vt_order = seq_ % 16 == 0 ? 1 : 0;
        int8_t *out_q    = nullptr;
        float out_q_inv  = 0.f;
        if (p->out_quant) {  // the last output: the context quantised as the folded Reformat layer would
            auto b8 = dynamic_cast<BlobInt8 *>(outputs.back());
            if (outputs.size() < 2 || !b8 || !b8->GetIntResource() || b8->GetIntResource()->scale_handle.GetDataCount() != 1 ||
                seq_ % 8 != 0)
                return Status(TNNERR_PARAM_ERR, "fused attention: the quantised output needs an int8 blob with one scale");
            out_q     = (int8_t *)Ptr(outputs.back());
            out_q_inv = (float)(1.0 / b8->GetIntResource()->scale_handle.force_to<float *>()[0]);
        }
        if (p->quant) {
            // int8 projections, requantised and dequantised in the GEMM epilogue, in the split layout
            char *vt = (char *)qkv + (size_t)T_ * 2 * H_ * es;
            ROCM_CALL(tnn_rocm_gemm_i8_qkv_split(Stream(), (int)dt, (const int8_t *)Ptr(inputs[0]), (const int8_t *)weight_,
                                                 (const int32_t *)bias_, (const float *)scale_, (const float *)dequant_, qkv,
                                                 vt, B_, seq_, p->heads, K_, vt_order));
            const long row = 2L * H_;
            ROCM_CALL(tnn_rocm_attention_vt_q8(Stream(), (int)dt, base, base + (size_t)H_ * es, vt, Ptr(outputs[0]), out_q,
                                               out_q_inv, B_, p->heads, seq_, p->head_dim, (long)seq_ * row, d, row,
                                               (long)seq_ * row, d, row, (long)p->heads * 64 * seq_, 64L * seq_, (long)seq_,
                                               (long)seq_ * H_, d, (long)H_, p->scale, mask, kv, vt_order));
            return TNN_OK;
        }
        if (seq_ % 8 == 0 && H_ % 64 == 0) {
            // projection writes Q|K row-major and V already transposed per head: the attention kernel then stages
            // V tiles with 16-byte copies
            char *vt = (char *)qkv + (size_t)T_ * 2 * H_ * es;
            if (p->ln_fold)
                ROCM_CALL(tnn_rocm_gemm_qkv_split_ln(Stream(), (int)dt, Ptr(inputs[0]), weight_, (const float *)bias_,
                                                     (const float *)colsum_, (const float *)gamma_, (const float *)beta_,
                                                     p->ln_eps, qkv, vt, p->ln_y ? Ptr(outputs[1]) : nullptr, (float *)stats,
                                                     (const float *)sums, blocks, B_, seq_, p->heads, H_, vt_order));
            else
                ROCM_CALL(tnn_rocm_gemm_qkv_split(Stream(), (int)dt, Ptr(inputs[0]), weight_, (const float *)bias_, qkv, vt,
                                                  B_, seq_, p->heads, H_, vt_order));
            const long row = 2L * H_;
            ROCM_CALL(tnn_rocm_attention_vt_q8(Stream(), (int)dt, base, base + (size_t)H_ * es, vt, Ptr(outputs[0]), out_q,
                                               out_q_inv, B_, p->heads, seq_, p->head_dim, (long)seq_ * row, d, row,
                                               (long)seq_ * row, d, row, (long)p->heads * 64 * seq_, 64L * seq_, (long)seq_,
                                               (long)seq_ * H_, d, (long)H_, p->scale, mask, kv, vt_order));
            return TNN_OK;
        }
        // sequence lengths that are not a multiple of 8 (only reachable by Instance::Reshape when a fold was decided
        // at another length): packed Q|K|V rows and the kernel that reads V row-major
        if (p->out_quant)
            return Status(TNNERR_PARAM_ERR, "fused attention: the quantised output needs a sequence length that is a multiple of 8");
        if (p->ln_fold)
            ROCM_CALL(tnn_rocm_gemm_ln(Stream(), (int)dt, Ptr(inputs[0]), weight_, (const float *)bias_, (const float *)colsum_,
                                       (const float *)gamma_, (const float *)beta_, p->ln_eps, qkv,
                                       p->ln_y ? Ptr(outputs[1]) : nullptr, (float *)stats, (const float *)sums, blocks, T_,
                                       3 * H_, H_, 0, nullptr));
        else
            ROCM_CALL(tnn_rocm_gemm(Stream(), (int)dt, 1, Ptr(inputs[0]), weight_, qkv, T_, 3 * H_, H_, H_, H_, 3 * H_, 1, 1, 1,
                                    TNN_ROCM_EPI_BIAS, (const float *)bias_, nullptr, 0));
        const long row = 3L * H_;
        ROCM_CALL(tnn_rocm_attention(Stream(), (int)dt, base, base + (size_t)H_ * es, base + (size_t)2 * H_ * es,
                                     Ptr(outputs[0]), B_, p->heads, seq_, p->head_dim, (long)seq_ * row, d, row,
                                     (long)seq_ * row, d, row, (long)seq_ * H_, d, (long)H_, p->scale, mask, kv));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr, *bias_ = nullptr, *scale_ = nullptr, *dequant_ = nullptr, *colsum_ = nullptr, *gamma_ = nullptr,
         *beta_ = nullptr;
    int H_ = 0, K_ = 0, T_ = 0, B_ = 0, seq_ = 0;
    bool mask_one_row_ = false;
};
REGISTER_ROCM_ACC(RocmFusedAttentionLayerAcc, LAYER_ROCM_FUSED_ATTENTION);

// ---- RocmFusedEmbedding ----------------------------------------------------------------------------------------
class RocmFusedEmbeddingLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto res = dynamic_cast<RocmFusedEmbeddingResource *>(resource_);
        CHECK_PARAM_NULL(res);
        if ((inputs.size() != 4 && inputs.size() != 5) || inputs[0]->GetBlobDesc().data_type != DATA_TYPE_INT32 ||
            inputs[1]->GetBlobDesc().data_type != DATA_TYPE_INT32 ||
            inputs[0]->GetBlobDesc().dims != inputs[1]->GetBlobDesc().dims)
            return Status(TNNERR_PARAM_ERR, "fused embedding: two int32 index blobs of equal shape, gamma and beta expected");
        n_pos_ids_ = 0;
        if (inputs.size() == 5) {  // position ids: the ids' shape, or one row [1,S] / [S] shared by the batch
            const int rows = DimsVectorUtils::Count(inputs[0]->GetBlobDesc().dims);
            n_pos_ids_     = DimsVectorUtils::Count(inputs[4]->GetBlobDesc().dims);
            if (inputs[4]->GetBlobDesc().data_type != DATA_TYPE_INT32 || n_pos_ids_ <= 0 || rows % n_pos_ids_ != 0 ||
                (n_pos_ids_ != rows && n_pos_ids_ != inputs[0]->GetBlobDesc().dims.back()))
                return Status(TNNERR_PARAM_ERR, "fused embedding: position ids must be int32 of the ids' shape or one row of it");
        }
        auto wd = res->word.GetBufferDims(), td = res->type.GetBufferDims(), pd = res->pos.GetBufferDims();
        auto id = inputs[0]->GetBlobDesc().dims;
        H_        = wd[1];
        pos_rows_ = pd[pd.size() - 2];
        // row t of the ids gets position t mod S.  The constant was matched at the shape the instance was created
        // with; after a reshape to a shorter sequence its first S rows are the positions 0..S-1.
        if (id.empty() || id.back() <= 0 || (n_pos_ids_ == 0 && id.back() > pos_rows_))
            return Status(TNNERR_PARAM_ERR, "fused embedding: the position constant does not cover the sequence length");
        period_ = id.back();
        vocab_ = wd[0], types_ = td[0];
        if (word_)
            return TNN_OK;
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        RETURN_ON_NEQ(UploadConverted(res->word.force_to<void *>(), (size_t)vocab_ * H_, DATA_TYPE_FLOAT, dt, &word_), TNN_OK);
        RETURN_ON_NEQ(UploadConverted(res->type.force_to<void *>(), (size_t)types_ * H_, DATA_TYPE_FLOAT, dt, &type_), TNN_OK);
        RETURN_ON_NEQ(UploadConverted(res->pos.force_to<void *>(), (size_t)pos_rows_ * H_, DATA_TYPE_FLOAT, dt, &pos_), TNN_OK);
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto p = dynamic_cast<RocmFusedEmbeddingParam *>(param_);
        Blob *gamma = In(inputs[2]), *beta = In(inputs[3]);
        if (gamma->GetBlobDesc().data_type != DATA_TYPE_FLOAT || beta->GetBlobDesc().data_type != DATA_TYPE_FLOAT ||
            DimsVectorUtils::Count(gamma->GetBlobDesc().dims) != H_ || DimsVectorUtils::Count(beta->GetBlobDesc().dims) != H_)
            return Status(TNNERR_PARAM_ERR, "fused embedding: gamma/beta must be fp32 vectors of the hidden size");
        const int rows = DimsVectorUtils::Count(inputs[0]->GetBlobDesc().dims);
        if (n_pos_ids_ > 0) {
            ROCM_CALL(tnn_rocm_embed_layernorm_pos(Stream(), (int)outputs[0]->GetBlobDesc().data_type,
                                                   (const int32_t *)Ptr(inputs[0]), (const int32_t *)Ptr(inputs[1]),
                                                   (const int32_t *)Ptr(inputs[4]), n_pos_ids_, word_, vocab_, type_, types_,
                                                   pos_, pos_rows_, (const float *)Ptr(gamma), (const float *)Ptr(beta),
                                                   p->eps, Ptr(outputs[0]), rows, H_, context_->ErrorFlag()));
            return TNN_OK;
        }
        ROCM_CALL(tnn_rocm_embed_layernorm(Stream(), (int)outputs[0]->GetBlobDesc().data_type, (const int32_t *)Ptr(inputs[0]),
                                           (const int32_t *)Ptr(inputs[1]), word_, vocab_, type_, types_, pos_, period_,
                                           (const float *)Ptr(gamma), (const float *)Ptr(beta), p->eps, Ptr(outputs[0]), rows,
                                           H_, context_->ErrorFlag()));
        return TNN_OK;
    }

protected:
    DataType ConstantBlobDataType(const std::vector<Blob *> &, int) override { return DATA_TYPE_FLOAT; }

private:
    void *word_ = nullptr, *type_ = nullptr, *pos_ = nullptr;
    int H_ = 0, period_ = 0, pos_rows_ = 0, vocab_ = 0, types_ = 0, n_pos_ids_ = 0;
};
REGISTER_ROCM_ACC(RocmFusedEmbeddingLayerAcc, LAYER_ROCM_FUSED_EMBEDDING);

// ---- RocmFusedLinearInt8 ---------------------------------------------------------------------------------------
// QuantizedInnerProduct (x86_inner_product_layer_acc.cc:274-288 -> X86GemvInt8) whose int8 result is read as float:
// y = float2int8((acc + bias) * w_scale / o_scale) * o_scale (+ residual), the value of
// QuantizedInnerProduct -> Reformat(int8->float) [-> Add], with the int8 value formed in registers only.
class RocmFusedLinearInt8LayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        if (weight_)
            return TNN_OK;
        auto p   = dynamic_cast<RocmFusedLinearInt8Param *>(param_);
        auto res = dynamic_cast<InnerProductLayerResource *>(resource_);
        CHECK_PARAM_NULL(p);
        if (!res)
            return Status(TNNERR_MODEL_ERR, "Error: InnerProductLayerResource is nil");
        const int N = p->num_output;
        const int K = DimsVectorUtils::Count(inputs[0]->GetBlobDesc().dims, p->axis);
        if ((long)res->weight_handle.GetDataCount() != (long)N * K || res->weight_handle.GetDataType() != DATA_TYPE_INT8)
            return Status(TNNERR_MODEL_ERR, "fused int8 linear: int8 weight of num_output x K expected");
        const DataType odt = outputs[0]->GetBlobDesc().data_type;
        if (inputs[0]->GetBlobDesc().data_type != DATA_TYPE_INT8 || (odt != DATA_TYPE_FLOAT && odt != DATA_TYPE_HALF))
            return Status(TNNERR_LAYER_ERR, "fused int8 linear: int8 input and fp32/fp16 output expected");
        if (p->has_residual && (inputs.size() != 2 || In(inputs[1])->GetBlobDesc().dims != outputs[0]->GetBlobDesc().dims ||
                                In(inputs[1])->GetBlobDesc().data_type != outputs[0]->GetBlobDesc().data_type))
            return Status(TNNERR_PARAM_ERR, "fused int8 linear: residual must have the output's shape and type");
        const float *w_scale = res->scale_handle.force_to<float *>();
        CHECK_PARAM_NULL(w_scale);
        const int n_w = res->scale_handle.GetDataCount();
        std::vector<float> scale(N);
        for (int i = 0; i < N; ++i)
            scale[i] = p->out_scale >= FLT_MIN ? w_scale[n_w == 1 ? 0 : i] / p->out_scale : 0.0f;
        RETURN_ON_NEQ(UploadConverted(res->weight_handle.force_to<void *>(), (size_t)N * K, DATA_TYPE_INT8, DATA_TYPE_INT8,
                                      &weight_), TNN_OK);
        RETURN_ON_NEQ(UploadConverted(scale.data(), (size_t)N, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &scale_), TNN_OK);
        if (p->has_bias && res->bias_handle.GetDataCount() == N)
            RETURN_ON_NEQ(UploadConverted(res->bias_handle.force_to<void *>(), (size_t)N, DATA_TYPE_INT32, DATA_TYPE_INT32,
                                          &bias_), TNN_OK);
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto p       = dynamic_cast<RocmFusedLinearInt8Param *>(param_);
        auto in_dims = inputs[0]->GetBlobDesc().dims;
        const int N = p->num_output, K = DimsVectorUtils::Count(in_dims, p->axis);
        const int rows = DimsVectorUtils::Count(in_dims, 0, p->axis);
        ROCM_CALL(tnn_rocm_gemm_i8_dequant_residual(Stream(), (const int8_t *)Ptr(inputs[0]), (const int8_t *)weight_,
                                                    (const int32_t *)bias_, (const float *)scale_, rows, N, K, K, K,
                                                    Ptr(outputs[0]), (int)outputs[0]->GetBlobDesc().data_type, N, p->out_scale,
                                                    p->has_residual ? Ptr(In(inputs[1])) : nullptr));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr, *bias_ = nullptr, *scale_ = nullptr;
};
REGISTER_ROCM_ACC(RocmFusedLinearInt8LayerAcc, LAYER_ROCM_FUSED_LINEAR_INT8);

// ---- RocmQuantLinearGelu ------------------------------------------------------------------------------------------
// QuantizedInnerProduct (x86_inner_product_layer_acc.cc:197-222: requantisation factor w_scale / o_scale as one host
// fp32 division, 0 below FLT_MIN) with the Reformat -> GELU -> Reformat chain that followed applied to its int8
// result as a table.  The table is produced once by the int8 GELU kernel itself on the 256 possible inputs.
class RocmQuantLinearGeluLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        if (weight_)
            return TNN_OK;
        auto p   = dynamic_cast<RocmQuantLinearGeluParam *>(param_);
        auto res = dynamic_cast<InnerProductLayerResource *>(resource_);
        auto out8 = dynamic_cast<BlobInt8 *>(outputs[0]);
        CHECK_PARAM_NULL(p);
        CHECK_PARAM_NULL(res);
        if (!out8 || !out8->GetIntResource() || out8->GetIntResource()->scale_handle.GetDataCount() != 1 ||
            inputs[0]->GetBlobDesc().data_type != DATA_TYPE_INT8 || res->weight_handle.GetDataType() != DATA_TYPE_INT8)
            return Status(TNNERR_PARAM_ERR, "quantised linear + GELU: int8 input, weights and a per-tensor output scale are required");
        const int N = p->num_output, K = DimsVectorUtils::Count(inputs[0]->GetBlobDesc().dims, p->axis);
        if ((long)res->weight_handle.GetDataCount() != (long)N * K)
            return Status(TNNERR_MODEL_ERR, "InnerProduct weight size does not match num_output x K");
        const float *w_scale = res->scale_handle.force_to<float *>();
        CHECK_PARAM_NULL(w_scale);
        const int n_w = res->scale_handle.GetDataCount();
        std::vector<float> scale(N);
        for (int i = 0; i < N; ++i)
            scale[i] = p->mid_scale >= FLT_MIN ? w_scale[n_w == 1 ? 0 : i] / p->mid_scale : 0.0f;
        RETURN_ON_NEQ(UploadConverted(res->weight_handle.force_to<void *>(), (size_t)N * K, DATA_TYPE_INT8, DATA_TYPE_INT8, &weight_),
                      TNN_OK);
        RETURN_ON_NEQ(UploadConverted(scale.data(), (size_t)N, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &scale_), TNN_OK);
        if (p->has_bias && res->bias_handle.GetDataCount() == N)
            RETURN_ON_NEQ(UploadConverted(res->bias_handle.force_to<void *>(), (size_t)N, DATA_TYPE_INT32, DATA_TYPE_INT32, &bias_),
                          TNN_OK);
        // the table: GELU chain of every int8 value, computed by the kernel the un-folded graph would run
        int8_t iota[256];
        for (int i = 0; i < 256; ++i)
            iota[i] = (int8_t)(i - 128);
        void *iota_dev = nullptr;
        RETURN_ON_NEQ(UploadConverted(iota, 256, DATA_TYPE_INT8, DATA_TYPE_INT8, &iota_dev), TNN_OK);
        RETURN_ON_NEQ(UploadConverted(iota, 256, DATA_TYPE_INT8, DATA_TYPE_INT8, &lut_), TNN_OK);
        const float s_out = out8->GetIntResource()->scale_handle.force_to<float *>()[0];
        ROCM_CALL(tnn_rocm_gelu_i8(Stream(), (const int8_t *)iota_dev, p->mid_scale, (float)(1.0 / s_out), (int8_t *)lut_, 256));
        ROCM_CALL(tnn_rocm_stream_sync(Stream()));
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto p = dynamic_cast<RocmQuantLinearGeluParam *>(param_);
        auto in_dims = inputs[0]->GetBlobDesc().dims;
        const int N = p->num_output, K = DimsVectorUtils::Count(in_dims, p->axis);
        const int rows = DimsVectorUtils::Count(in_dims, 0, p->axis);
        ROCM_CALL(tnn_rocm_gemm_i8_lut(Stream(), (const int8_t *)Ptr(inputs[0]), (const int8_t *)weight_, (const int32_t *)bias_,
                                       (const float *)scale_, (int8_t *)Ptr(outputs[0]), rows, N, K, K, K, N, (const int8_t *)lut_));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr, *bias_ = nullptr, *scale_ = nullptr, *lut_ = nullptr;
};
REGISTER_ROCM_ACC(RocmQuantLinearGeluLayerAcc, LAYER_ROCM_QUANT_LINEAR_GELU);

// ---- RocmGeluInt8 -----------------------------------------------------------------------------------------------
// Reformat(int8->float) -> GELU -> Reformat(float->int8) on int8 blobs in one pass: q_out =
// float2int8(gelu(q_in * s_in) * float(1.0 / s_out)) (x86_compute_int8.cc:1193-1318, cpu_gelu_layer_acc.cc:42-45).
class RocmGeluInt8LayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto in8 = dynamic_cast<BlobInt8 *>(inputs[0]), out8 = dynamic_cast<BlobInt8 *>(outputs[0]);
        if (!in8 || !out8 || !in8->GetIntResource() || !out8->GetIntResource() ||
            in8->GetIntResource()->scale_handle.GetDataCount() != 1 || out8->GetIntResource()->scale_handle.GetDataCount() != 1)
            return Status(TNNERR_LAYER_ERR, "int8 GELU needs per-tensor blob scales on both sides");
        float s_in  = in8->GetIntResource()->scale_handle.force_to<float *>()[0];
        float s_out = out8->GetIntResource()->scale_handle.force_to<float *>()[0];
        ROCM_CALL(tnn_rocm_gelu_i8(Stream(), (const int8_t *)Ptr(inputs[0]), s_in, (float)(1.0 / s_out), (int8_t *)Ptr(outputs[0]),
                                   (size_t)DimsVectorUtils::Count(inputs[0]->GetBlobDesc().dims)));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmGeluInt8LayerAcc, LAYER_ROCM_GELU_INT8);

}  // namespace TNN_NS
