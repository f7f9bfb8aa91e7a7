// extern "C" surface of include/tllm_stack_api.h: the ragged-batch step executor for run-time described decoder stacks.
//
// One step = embedding -> the layer runs in order -> final norm + head on the wanted rows -> arg-max.  A layer run is
//   h1, h2 = norm1(x), norm2(x)                                  one launch (the two norms share the normalised row)
//   P1 = h1 [Wq; Wk; Wv; Wrg1]^T   (hgrn2: [Wq; Wf; Wv; Wrg1])    one product: everything that reads h1
//   ctx = mixer(P1)                                              rotary + cache append + attention | recurrence + head norm
//   x += sigmoid(P1[rg1] + b1) * (ctx Wo^T)                      product with the gated-residual seam in its epilogue
//   P2 = h2 [Wgate; Wup; Wrg2]^T ; a = gelu(P2[gate]) * P2[up]
//   x += sigmoid(P2[rg2] + b2) * (a Wdown^T)
// on the packed rows of the step.  The residual stream x is fp32 in both element types.
#include "../../../include/tllm_stack_api.h"
#include "../kernels/stack_kernels.h"
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

using namespace tllm;
using namespace tllm::kernels;

namespace
{

struct HostTensor
{
    std::vector<int64_t> dims;
    std::vector<float> v; // every weight passes through fp32 on the host (bfloat16 -> fp32 is exact)
    int64_t numel() const
    {
        int64_t n = 1;
        for (auto d : dims)
            n *= d;
        return n;
    }
};

enum MixerKind
{
    MIX_ATTENTION = 0,
    MIX_HGRN2 = 1
};

struct Layer
{
    int kind = MIX_ATTENTION;
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0, maps = 1, ff = 0, head_norm = 0;
    double diff = 0, scale = 1, softcap = 0;
    int rot_dims = 0;
    double rot_base = 10000, rot_factor = 0, rot_original = 0, rot_fast = 0, rot_slow = 0;
    // derived
    int n_q = 0, n_k = 0, n_v = 0, n_mix = 0, n_ctx = 0; // columns of P1: q | k (or f) | v | rg1
    float lambda = 0.f, mscale = 1.f;
    // device
    void *w_mix = nullptr, *w_o = nullptr, *w_gu = nullptr, *w_down = nullptr;
    float *norm1 = nullptr, *norm2 = nullptr, *rg1_b = nullptr, *rg2_b = nullptr, *f_bias = nullptr, *lower = nullptr, *hnorm = nullptr,
          *freq = nullptr;
};

struct Run
{
    int layer = 0, pass = 0;
    bool enters_pass = false;
    void *k_pool = nullptr, *v_pool = nullptr; // attention
    float* state = nullptr;                    // hgrn2
};

} // namespace

struct tllm_stack
{
    std::map<std::string, std::string> cfg;
    std::map<std::string, HostTensor> host;
    int dtype = DT_BF16, es = 2;
    int width = 0, vocab = 0, groups = 1, page = 64, blocks = 0, slots = 0, taps = 0;
    int loop_start = 0, loop_stop = 0, loop_times = 1;
    float eps = 1e-5f, emb_scale = 1.f;
    std::vector<Layer> layers;
    std::vector<Run> runs;
    void *embed = nullptr, *head = nullptr;
    float *final_norm = nullptr, *loop_step = nullptr, *attn_ws = nullptr;
    bool finalized = false;
    int64_t weight_bytes = 0;
    std::vector<void*> owned;
    // scratch, grown to the largest step seen
    int cap_tokens = 0, cap_want = 0, cap_ints = 0;
    float *x = nullptr, *x0 = nullptr, *o32 = nullptr, *logits = nullptr, *tap = nullptr;
    void *h1 = nullptr, *h2 = nullptr, *proj = nullptr, *q = nullptr, *ctx = nullptr, *act = nullptr, *hw = nullptr;
    int32_t *ints = nullptr, *ids_out = nullptr, *pinned = nullptr;
    int max_proj = 0, max_q = 0, max_ctx = 0, max_ff = 0;
    int tap_tokens = 0;

    ~tllm_stack()
    {
        for (void* p : owned)
            (void) hipFree(p);
        free_scratch();
        if (pinned)
            (void) hipHostFree(pinned);
    }
    void free_scratch()
    {
        void* all[] = {x, x0, o32, logits, tap, h1, h2, proj, q, ctx, act, hw, ints, ids_out};
        for (void* p : all)
            if (p)
                (void) hipFree(p);
        x = x0 = o32 = logits = tap = nullptr;
        h1 = h2 = proj = q = ctx = act = hw = nullptr;
        ints = ids_out = nullptr;
    }
};

namespace
{

#define HIP_OK(call)                                                                                                              \
    do                                                                                                                              \
    {                                                                                                                               \
        const hipError_t e_ = (call);                                                                                               \
        if (e_ != hipSuccess)                                                                                                       \
        {                                                                                                                           \
            set_error("stack engine: %s failed: %s", #call, hipGetErrorString(e_));                                               \
            return -1;                                                                                                              \
        }                                                                                                                           \
    } while (0)

inline uint16_t host_f2bf(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t) ((u >> 16) | 0x40u);
    return (uint16_t) ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

double getd(const tllm_stack* s, const std::string& k, double dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : std::atof(it->second.c_str());
}
int geti(const tllm_stack* s, const std::string& k, int dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : std::atoi(it->second.c_str());
}
std::string gets(const tllm_stack* s, const std::string& k, const std::string& dflt)
{
    auto it = s->cfg.find(k);
    return it == s->cfg.end() ? dflt : it->second;
}

// rows of several [n_i, K] host matrices stacked into one device matrix of the engine's element type
int upload_rows(tllm_stack* s, const std::vector<const HostTensor*>& parts, void** out)
{
    int64_t n = 0;
    for (auto* t : parts)
        n += t->numel();
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, (size_t) (n ? n : 1) * s->es));
    s->owned.push_back(d);
    s->weight_bytes += n * s->es;
    int64_t off = 0;
    std::vector<uint16_t> tmp;
    for (auto* t : parts)
    {
        if (s->dtype == DT_FLOAT)
            HIP_OK(hipMemcpy((char*) d + off * 4, t->v.data(), t->v.size() * 4, hipMemcpyHostToDevice));
        else
        {
            tmp.resize(t->v.size());
            for (size_t i = 0; i < tmp.size(); ++i)
                tmp[i] = host_f2bf(t->v[i]);
            HIP_OK(hipMemcpy((char*) d + off * 2, tmp.data(), tmp.size() * 2, hipMemcpyHostToDevice));
        }
        off += t->numel();
    }
    *out = d;
    return 0;
}

int upload_f32(tllm_stack* s, const float* v, size_t n, float** out)
{
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, (n ? n : 1) * 4));
    s->owned.push_back(d);
    s->weight_bytes += (int64_t) n * 4;
    HIP_OK(hipMemcpy(d, v, n * 4, hipMemcpyHostToDevice));
    *out = (float*) d;
    return 0;
}

const HostTensor* need(tllm_stack* s, const std::string& name, std::initializer_list<int64_t> dims)
{
    auto it = s->host.find(name);
    if (it == s->host.end())
    {
        set_error("tllm_stack_finalize: tensor %s is missing", name.c_str());
        return nullptr;
    }
    const std::vector<int64_t> want(dims);
    if (it->second.dims != want)
    {
        std::string have, w;
        for (auto d : it->second.dims)
            have += std::to_string(d) + " ";
        for (auto d : want)
            w += std::to_string(d) + " ";
        set_error("tllm_stack_finalize: tensor %s has shape [ %s], the configuration asks for [ %s]", name.c_str(), have.c_str(), w.c_str());
        return nullptr;
    }
    return &it->second;
}

int alloc_zero(tllm_stack* s, size_t bytes, void** out)
{
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, bytes ? bytes : 16));
    s->owned.push_back(d);
    HIP_OK(hipMemset(d, 0, bytes ? bytes : 16));
    *out = d;
    return 0;
}

int ensure_scratch(tllm_stack* s, int tokens, int want, int n_ints)
{
    if (tokens > s->cap_tokens || want > s->cap_want || n_ints > s->cap_ints)
    {
        HIP_OK(hipDeviceSynchronize());
        s->free_scratch();
        if (s->pinned)
        {
            (void) hipHostFree(s->pinned);
            s->pinned = nullptr;
        }
        const size_t T = (size_t) std::max(tokens, s->cap_tokens), W = (size_t) std::max(want, s->cap_want);
        const size_t NI = (size_t) std::max(n_ints, s->cap_ints);
        const size_t es = s->es, wd = s->width;
        HIP_OK(hipMalloc((void**) &s->x, T * wd * 4));
        HIP_OK(hipMalloc((void**) &s->x0, T * wd * 4));
        HIP_OK(hipMalloc((void**) &s->o32, T * std::max(s->max_ctx, 1) * 4));
        HIP_OK(hipMalloc((void**) &s->logits, W * s->vocab * 4));
        HIP_OK(hipMalloc(&s->h1, T * wd * es));
        HIP_OK(hipMalloc(&s->h2, T * wd * es));
        HIP_OK(hipMalloc(&s->proj, T * std::max(s->max_proj, 1) * es));
        HIP_OK(hipMalloc(&s->q, T * std::max(s->max_q, 1) * es));
        HIP_OK(hipMalloc(&s->ctx, T * std::max(s->max_ctx, 1) * es));
        HIP_OK(hipMalloc(&s->act, T * std::max(s->max_ff, 1) * es));
        HIP_OK(hipMalloc(&s->hw, W * wd * es));
        HIP_OK(hipMalloc((void**) &s->ints, NI * 4));
        HIP_OK(hipMalloc((void**) &s->ids_out, W * 4));
        HIP_OK(hipHostMalloc((void**) &s->pinned, NI * 4, hipHostMallocDefault));
        if (s->taps)
            HIP_OK(hipMalloc((void**) &s->tap, s->runs.size() * T * wd * 4));
        s->cap_tokens = (int) T;
        s->cap_want = (int) W;
        s->cap_ints = (int) NI;
    }
    return 0;
}

} // namespace

extern "C" {

tllm_stack_t tllm_stack_create(const char* config_text)
{
    if (!config_text)
    {
        set_error("tllm_stack_create: no configuration");
        return nullptr;
    }
    auto* s = new tllm_stack();
    std::string text(config_text);
    size_t at = 0;
    while (at < text.size())
    {
        size_t nl = text.find('\n', at);
        if (nl == std::string::npos)
            nl = text.size();
        const std::string line = text.substr(at, nl - at);
        at = nl + 1;
        const size_t eq = line.find('=');
        if (eq == std::string::npos)
            continue;
        s->cfg[line.substr(0, eq)] = line.substr(eq + 1);
    }
    const std::string dt = gets(s, "dtype", "bfloat16");
    if (dt == "bfloat16")
        s->dtype = DT_BF16, s->es = 2;
    else if (dt == "float32")
        s->dtype = DT_FLOAT, s->es = 4;
    else
    {
        set_error("tllm_stack_create: dtype %s (bfloat16 or float32)", dt.c_str());
        delete s;
        return nullptr;
    }
    s->width = geti(s, "width", 0);
    s->vocab = geti(s, "vocab", 0);
    s->groups = geti(s, "norm_groups", 1);
    s->eps = (float) getd(s, "norm_eps", 1e-5);
    s->emb_scale = (float) getd(s, "embedding_scale", 1.0);
    s->page = geti(s, "page_size", 64);
    s->blocks = geti(s, "num_blocks", 0);
    s->slots = geti(s, "num_slots", 0);
    s->taps = geti(s, "debug_taps", 0);
    s->loop_start = geti(s, "loop_start", 0);
    s->loop_stop = geti(s, "loop_stop", 0);
    s->loop_times = geti(s, "loop_times", 1);
    const int L = geti(s, "num_layers", 0);
    auto fail = [&](const char* why) {
        set_error("tllm_stack_create: %s", why);
        delete s;
        return (tllm_stack_t) nullptr;
    };
    if (s->width < 1 || s->vocab < 1 || L < 1)
        return fail("width, vocab and num_layers must be positive");
    if (s->groups < 1 || s->width % s->groups)
        return fail("width must split into norm_groups equal parts");
    if (s->page < 1 || s->blocks < 1 || s->slots < 1)
        return fail("page_size, num_blocks and num_slots must be positive");
    if (s->loop_times < 1 || s->loop_start < 0 || s->loop_stop < s->loop_start || s->loop_stop > L)
        return fail("the loop must satisfy 0 <= loop_start <= loop_stop <= num_layers, loop_times >= 1");
    s->layers.resize(L);
    for (int i = 0; i < L; ++i)
    {
        Layer& l = s->layers[i];
        const std::string p = "layer." + std::to_string(i) + ".";
        const std::string kind = gets(s, p + "type", "");
        if (kind == "attention")
            l.kind = MIX_ATTENTION;
        else if (kind == "hgrn2")
            l.kind = MIX_HGRN2;
        else
        {
            set_error("tllm_stack_create: layer %d has mixer type '%s' (attention | hgrn2)", i, kind.c_str());
            delete s;
            return nullptr;
        }
        l.heads = geti(s, p + "heads", 0);
        l.dim = geti(s, p + "dim", 0);
        l.vdim = geti(s, p + "vdim", l.dim);
        l.ff = geti(s, p + "ff", 0);
        if (l.heads < 1 || l.dim < 1 || l.vdim < 1 || l.ff < 0)
            return fail("a layer needs heads, dim and vdim");
        l.n_ctx = l.heads * l.vdim;
        if (l.kind == MIX_ATTENTION)
        {
            l.kv_heads = geti(s, p + "kv_heads", l.heads);
            l.maps = geti(s, p + "maps", 1);
            l.diff = getd(s, p + "diff", 0);
            l.scale = getd(s, p + "scale", 1.0 / std::sqrt((double) l.dim));
            l.softcap = getd(s, p + "softcap", 0);
            l.head_norm = geti(s, p + "head_norm", 0);
            l.rot_dims = geti(s, p + "rot_dims", 0);
            l.rot_base = getd(s, p + "rot_base", 10000);
            l.rot_factor = getd(s, p + "rot_factor", 0);
            l.rot_original = getd(s, p + "rot_original", 0);
            l.rot_fast = getd(s, p + "rot_fast", 0);
            l.rot_slow = getd(s, p + "rot_slow", 0);
            if (l.kv_heads < 1 || l.heads % l.kv_heads || l.maps < 1 || l.maps > 2 || (l.dim & 1) || (l.rot_dims & 1) || l.rot_dims > l.dim)
                return fail("attention: heads must be a multiple of kv_heads, maps 1 or 2, dim and rot_dims even, rot_dims <= dim");
            l.n_q = l.heads * l.maps * l.dim;
            l.n_k = l.kv_heads * l.maps * l.dim;
            l.n_v = l.kv_heads * l.vdim;
        }
        else
        {
            if (!stack_hgrn2_serves(l.dim, l.vdim))
                return fail("hgrn2: dim up to 512");
            l.n_q = l.heads * l.dim;
            l.n_k = l.heads * l.dim; // forget gate
            l.n_v = l.heads * l.vdim;
        }
        l.n_mix = l.n_q + l.n_k + l.n_v + s->width;
        s->max_proj = std::max(s->max_proj, std::max(l.n_mix, 2 * l.ff + s->width));
        s->max_q = std::max(s->max_q, l.n_q);
        s->max_ctx = std::max(s->max_ctx, l.n_ctx);
        s->max_ff = std::max(s->max_ff, l.ff);
    }
    // execution order
    auto add = [&](int layer, int pass, bool enters) {
        Run r;
        r.layer = layer;
        r.pass = pass;
        r.enters_pass = enters;
        s->runs.push_back(r);
    };
    const bool looped = s->loop_stop > s->loop_start;
    for (int i = 0; i < (looped ? s->loop_start : L); ++i)
        add(i, 0, false);
    if (looped)
    {
        for (int t = 0; t < s->loop_times; ++t)
            for (int i = s->loop_start; i < s->loop_stop; ++i)
                add(i, t, i == s->loop_start);
        for (int i = s->loop_stop; i < L; ++i)
            add(i, 0, false);
    }
    return s;
}

int32_t tllm_stack_set_tensor(tllm_stack_t s, const char* name, int32_t dtype, const int64_t* dims, int32_t nbDims, const void* data)
{
    if (!s || !name || !data || nbDims < 0 || nbDims > 4 || s->finalized)
    {
        set_error("tllm_stack_set_tensor: bad arguments (or the engine is already finalized)");
        return -1;
    }
    HostTensor t;
    for (int i = 0; i < nbDims; ++i)
        t.dims.push_back(dims[i]);
    const int64_t n = t.numel();
    t.v.resize((size_t) n);
    if (dtype == DT_FLOAT)
        std::memcpy(t.v.data(), data, (size_t) n * 4);
    else if (dtype == DT_BF16)
    {
        const uint16_t* b = static_cast<const uint16_t*>(data);
        for (int64_t i = 0; i < n; ++i)
        {
            const uint32_t u = (uint32_t) b[i] << 16;
            std::memcpy(&t.v[(size_t) i], &u, 4);
        }
    }
    else
    {
        set_error("tllm_stack_set_tensor(%s): dtype %d (0 = fp32, 7 = bfloat16)", name, dtype);
        return -1;
    }
    s->host[name] = std::move(t);
    return 0;
}

int32_t tllm_stack_finalize(tllm_stack_t s)
{
    if (!s || s->finalized)
    {
        set_error("tllm_stack_finalize: no engine, or finalized twice");
        return -1;
    }
    const int64_t Wd = s->width;
    const HostTensor* t = need(s, "embed", {s->vocab, Wd});
    if (!t || upload_rows(s, {t}, &s->embed))
        return -1;
    t = need(s, "head", {s->vocab, Wd});
    if (!t || upload_rows(s, {t}, &s->head))
        return -1;
    t = need(s, "final.norm", {Wd});
    if (!t || upload_f32(s, t->v.data(), t->v.size(), &s->final_norm))
        return -1;
    if (s->loop_stop > s->loop_start)
    {
        t = need(s, "loop.step", {s->loop_times, Wd});
        if (!t || upload_f32(s, t->v.data(), t->v.size(), &s->loop_step))
            return -1;
    }
    for (size_t i = 0; i < s->layers.size(); ++i)
    {
        Layer& l = s->layers[i];
        const std::string p = "l" + std::to_string(i) + ".";
        auto vec = [&](const std::string& n, int64_t len, float** out) {
            const HostTensor* v = need(s, p + n, {len});
            return (!v || upload_f32(s, v->v.data(), v->v.size(), out)) ? -1 : 0;
        };
        if (vec("norm1", Wd, &l.norm1) || vec("rg1.b", Wd, &l.rg1_b))
            return -1;
        const HostTensor* rg1 = need(s, p + "rg1", {Wd, Wd});
        const HostTensor* wq = need(s, p + "mix.q", {l.n_q, Wd});
        const HostTensor* wk = need(s, p + (l.kind == MIX_ATTENTION ? "mix.k" : "mix.f"), {l.n_k, Wd});
        const HostTensor* wv = need(s, p + "mix.v", {l.n_v, Wd});
        const HostTensor* wo = need(s, p + "mix.o", {Wd, l.n_ctx});
        if (!rg1 || !wq || !wk || !wv || !wo)
            return -1;
        if (upload_rows(s, {wq, wk, wv, rg1}, &l.w_mix) || upload_rows(s, {wo}, &l.w_o))
            return -1;
        if (l.kind == MIX_ATTENTION)
        {
            std::vector<float> fr((size_t) std::max(l.rot_dims / 2, 1));
            l.mscale = stack_rope_freqs(fr.data(), l.rot_dims, l.rot_base, l.rot_factor, l.rot_original, l.rot_fast, l.rot_slow);
            if (upload_f32(s, fr.data(), fr.size(), &l.freq))
                return -1;
            l.lambda = 0.f;
            if (l.maps == 2)
            {
                const HostTensor *a1 = need(s, p + "mix.lq1", {l.dim}), *b1 = need(s, p + "mix.lk1", {l.dim}),
                                 *a2 = need(s, p + "mix.lq2", {l.dim}), *b2 = need(s, p + "mix.lk2", {l.dim});
                if (!a1 || !b1 || !a2 || !b2)
                    return -1;
                float d1 = 0.f, d2 = 0.f;
                for (int d = 0; d < l.dim; ++d)
                {
                    d1 += a1->v[d] * b1->v[d];
                    d2 += a2->v[d] * b2->v[d];
                }
                l.lambda = std::exp(d1) - std::exp(d2) + (float) l.diff;
            }
        }
        else
        {
            if (vec("mix.f.b", l.n_k, &l.f_bias) || vec("mix.lower", l.n_k, &l.lower) || vec("mix.norm", l.vdim, &l.hnorm))
                return -1;
        }
        if (l.ff > 0)
        {
            if (vec("norm2", Wd, &l.norm2) || vec("rg2.b", Wd, &l.rg2_b))
                return -1;
            const HostTensor* rg2 = need(s, p + "rg2", {Wd, Wd});
            const HostTensor* wg = need(s, p + "mlp.gate", {l.ff, Wd});
            const HostTensor* wu = need(s, p + "mlp.up", {l.ff, Wd});
            const HostTensor* wd = need(s, p + "mlp.down", {Wd, l.ff});
            if (!rg2 || !wg || !wu || !wd)
                return -1;
            if (upload_rows(s, {wg, wu, rg2}, &l.w_gu) || upload_rows(s, {wd}, &l.w_down))
                return -1;
        }
    }
    size_t ws_floats = 0;
    for (const Layer& l : s->layers)
        if (l.kind == MIX_ATTENTION)
            ws_floats = std::max(ws_floats, stack_attn_workspace_floats(l.heads, l.maps, l.vdim));
    if (ws_floats)
    {
        void* ws = nullptr;
        if (alloc_zero(s, ws_floats * 4, &ws))
            return -1;
        s->attn_ws = (float*) ws;
    }
    for (Run& r : s->runs)
    {
        const Layer& l = s->layers[r.layer];
        if (l.kind == MIX_ATTENTION)
        {
            if (alloc_zero(s, (size_t) s->blocks * l.kv_heads * l.maps * s->page * l.dim * s->es, &r.k_pool)
                || alloc_zero(s, (size_t) s->blocks * l.kv_heads * s->page * l.vdim * s->es, &r.v_pool))
                return -1;
        }
        else
        {
            void* st = nullptr;
            if (alloc_zero(s, (size_t) s->slots * l.heads * l.dim * l.vdim * 4, &st))
                return -1;
            r.state = (float*) st;
        }
    }
    s->host.clear();
    s->finalized = true;
    return 0;
}

int32_t tllm_stack_step(tllm_stack_t s, const tllm_stack_batch_t* b, float* logits_out, int32_t* next_ids_out, void* stream_v)
{
    if (!s || !s->finalized || !b)
    {
        set_error("tllm_stack_step: the engine is not finalized");
        return -1;
    }
    hipStream_t stream = (hipStream_t) stream_v;
    const int T = b->n_tokens, E = b->n_entries, NW = b->n_want, MB = b->max_blocks;
    if (T < 1 || E < 1 || NW < 0 || MB < 1 || !b->tokens || !b->ent_count || !b->ent_pos0 || !b->ent_slot || !b->block_table
        || (NW > 0 && !b->want_rows))
    {
        set_error("tllm_stack_step: empty batch or missing array");
        return -1;
    }
    // ---- every index the kernels will follow is checked here
    int64_t sum = 0;
    int max_count = 0, max_ctx = 0;
    for (int e = 0; e < E; ++e)
    {
        const int c = b->ent_count[e], p0 = b->ent_pos0[e], sl = b->ent_slot[e];
        if (c < 1 || p0 < 0 || sl < 0 || sl >= s->slots)
        {
            set_error("tllm_stack_step: entry %d has count %d, pos0 %d, slot %d (slots: %d)", e, c, p0, sl, s->slots);
            return -1;
        }
        for (int e2 = 0; e2 < e; ++e2)
            if (b->ent_slot[e2] == sl)
            {
                set_error("tllm_stack_step: entries %d and %d share slot %d", e2, e, sl);
                return -1;
            }
        const int nb = (p0 + c + s->page - 1) / s->page;
        if (nb > MB)
        {
            set_error("tllm_stack_step: entry %d needs %d blocks, its table has %d", e, nb, MB);
            return -1;
        }
        for (int j = 0; j < nb; ++j)
        {
            const int id = b->block_table[(size_t) e * MB + j];
            if (id < 0 || id >= s->blocks)
            {
                set_error("tllm_stack_step: entry %d, block %d of its table is %d (pool: %d blocks)", e, j, id, s->blocks);
                return -1;
            }
        }
        sum += c;
        max_count = std::max(max_count, c);
        max_ctx = std::max(max_ctx, p0 + c);
    }
    if (sum != T)
    {
        set_error("tllm_stack_step: the entries hold %lld tokens, the batch %d", (long long) sum, T);
        return -1;
    }
    for (int t = 0; t < T; ++t)
        if (b->tokens[t] < 0 || b->tokens[t] >= s->vocab)
        {
            set_error("tllm_stack_step: token %d at row %d is outside the vocabulary of %d", b->tokens[t], t, s->vocab);
            return -1;
        }
    for (int i = 0; i < NW; ++i)
        if (b->want_rows[i] < 0 || b->want_rows[i] >= T)
        {
            set_error("tllm_stack_step: wanted row %d is outside the batch of %d", b->want_rows[i], T);
            return -1;
        }
    // ---- metadata: one packed int32 image, one copy
    const size_t n_ints = (size_t) 3 * T + (size_t) 4 * E + (size_t) E * MB + NW;
    if (ensure_scratch(s, T, std::max(NW, 1), (int) n_ints))
        return -1;
    int32_t* h = s->pinned;
    int32_t *h_tok = h, *h_tent = h + T, *h_tpos = h + 2 * T, *h_first = h + 3 * T, *h_count = h_first + E, *h_pos0 = h_count + E,
            *h_slot = h_pos0 + E, *h_table = h_slot + E, *h_want = h_table + (size_t) E * MB;
    std::memcpy(h_tok, b->tokens, (size_t) T * 4);
    int row = 0;
    for (int e = 0; e < E; ++e)
    {
        h_first[e] = row;
        h_count[e] = b->ent_count[e];
        h_pos0[e] = b->ent_pos0[e];
        h_slot[e] = b->ent_slot[e];
        for (int i = 0; i < b->ent_count[e]; ++i, ++row)
        {
            h_tent[row] = e;
            h_tpos[row] = b->ent_pos0[e] + i;
        }
        const int nb = (b->ent_pos0[e] + b->ent_count[e] + s->page - 1) / s->page;
        for (int j = 0; j < MB; ++j)
            h_table[(size_t) e * MB + j] = j < nb ? b->block_table[(size_t) e * MB + j] : 0;
    }
    for (int i = 0; i < NW; ++i)
        h_want[i] = b->want_rows[i];
    HIP_OK(hipMemcpyAsync(s->ints, h, n_ints * 4, hipMemcpyHostToDevice, stream));
    const int32_t* d = s->ints;
    const int32_t *d_tok = d, *d_tent = d + T, *d_tpos = d + 2 * T, *d_first = d + 3 * T, *d_count = d_first + E, *d_pos0 = d_count + E,
                  *d_slot = d_pos0 + E, *d_table = d_slot + E, *d_want = d_table + (size_t) E * MB;

    const int Wd = s->width;
    const bool looped = s->loop_stop > s->loop_start;
    if (launch_stack_embed(s->x, looped && s->loop_times > 1 ? s->x0 : nullptr, d_tok, s->embed, s->dtype, T, Wd, s->vocab, s->emb_scale, stream))
        return -1;
    s->tap_tokens = T;
    for (size_t ri = 0; ri < s->runs.size(); ++ri)
    {
        const Run& r = s->runs[ri];
        const Layer& l = s->layers[r.layer];
        if (r.enters_pass
            && launch_stack_pass_entry(s->x, r.pass > 0 ? s->x0 : nullptr, s->loop_step + (size_t) r.pass * Wd, T, Wd, stream))
            return -1;
        if (launch_stack_group_rmsnorm(s->h1, l.ff > 0 ? s->h2 : nullptr, s->x, nullptr, l.norm1, l.norm2, s->dtype, T, Wd, s->groups, s->eps,
                stream))
            return -1;
        StackGemmParams g;
        g.dtype = s->dtype;
        g.M = T;
        g.N = l.n_mix;
        g.K = Wd;
        g.a = s->h1;
        g.lda = Wd;
        g.w = l.w_mix;
        g.c = s->proj;
        g.ldc = l.n_mix;
        if (launch_stack_gemm(g, stream))
            return -1;
        if (l.kind == MIX_ATTENTION)
        {
            StackAttnParams a;
            a.dtype = s->dtype;
            a.tokens = T;
            a.entries = E;
            a.heads = l.heads;
            a.kv_heads = l.kv_heads;
            a.maps = l.maps;
            a.dim = l.dim;
            a.vdim = l.vdim;
            a.rot_dims = l.rot_dims;
            a.freq = l.freq;
            a.mscale = l.mscale;
            a.scale = (float) l.scale;
            a.softcap = (float) l.softcap;
            a.lambda = l.lambda;
            a.out_scale = (float) (1.0 - l.diff);
            a.eps = s->eps;
            a.head_norm = l.head_norm;
            a.proj = s->proj;
            a.ldp = l.n_mix;
            a.q = s->q;
            a.k_pool = r.k_pool;
            a.v_pool = r.v_pool;
            a.page = s->page;
            a.max_blocks = MB;
            a.block_table = d_table;
            a.tok_entry = d_tent;
            a.tok_pos = d_tpos;
            a.ent_first = d_first;
            a.ent_count = d_count;
            a.ent_pos0 = d_pos0;
            a.max_count = max_count;
            a.max_context = max_ctx;
            a.out = s->ctx;
            a.split_ws = s->attn_ws;
            if (launch_stack_rope_kv(a, stream) || launch_stack_attention(a, stream))
                return -1;
        }
        else
        {
            StackHgrnParams hp;
            hp.dtype = s->dtype;
            hp.tokens = T;
            hp.entries = E;
            hp.heads = l.heads;
            hp.dim = l.dim;
            hp.vdim = l.vdim;
            hp.proj = s->proj;
            hp.ldp = l.n_mix;
            hp.f_bias = l.f_bias;
            hp.lower = l.lower;
            hp.norm_w = l.hnorm;
            hp.eps = s->eps;
            hp.state = r.state;
            hp.ent_slot = d_slot;
            hp.ent_first = d_first;
            hp.ent_count = d_count;
            hp.ent_pos0 = d_pos0;
            hp.max_count = max_count;
            hp.o32 = s->o32;
            hp.out = s->ctx;
            if (launch_stack_hgrn2(hp, stream))
                return -1;
        }
        // x += sigmoid(P1[rg1] + b1) * (ctx Wo^T)
        StackGemmParams o;
        o.dtype = s->dtype;
        o.M = T;
        o.N = Wd;
        o.K = l.n_ctx;
        o.a = s->ctx;
        o.lda = l.n_ctx;
        o.w = l.w_o;
        o.resid = s->x;
        o.ldr = Wd;
        o.gate = (const char*) s->proj + (size_t) (l.n_q + l.n_k + l.n_v) * s->es;
        o.ldg = l.n_mix;
        o.gate_bias = l.rg1_b;
        if (l.ff > 0)
        {
            // the feed-forward reads the same x as the mixer: its projection runs before the mixer's update lands (h2 is ready)
            StackGemmParams u;
            u.dtype = s->dtype;
            u.M = T;
            u.N = 2 * l.ff + Wd;
            u.K = Wd;
            u.a = s->h2;
            u.lda = Wd;
            u.w = l.w_gu;
            u.c = s->proj; // P1's columns are consumed once the mixer and the O product have run: keep the order below
            u.ldc = u.N;
            if (launch_stack_gemm(o, stream))
                return -1;
            if (launch_stack_gemm(u, stream) || launch_stack_gelu_gate(s->act, s->proj, s->dtype, T, l.ff, u.N, stream))
                return -1;
            StackGemmParams dn;
            dn.dtype = s->dtype;
            dn.M = T;
            dn.N = Wd;
            dn.K = l.ff;
            dn.a = s->act;
            dn.lda = l.ff;
            dn.w = l.w_down;
            dn.resid = s->x;
            dn.ldr = Wd;
            dn.gate = (const char*) s->proj + (size_t) (2 * l.ff) * s->es;
            dn.ldg = u.N;
            dn.gate_bias = l.rg2_b;
            if (launch_stack_gemm(dn, stream))
                return -1;
        }
        else if (launch_stack_gemm(o, stream))
            return -1;
        if (s->taps)
            HIP_OK(hipMemcpyAsync(s->tap + ri * (size_t) T * Wd, s->x, (size_t) T * Wd * 4, hipMemcpyDeviceToDevice, stream));
    }
    if (NW > 0)
    {
        if (launch_stack_group_rmsnorm(s->hw, nullptr, s->x, d_want, s->final_norm, nullptr, s->dtype, NW, Wd, s->groups, s->eps, stream))
            return -1;
        StackGemmParams hd;
        hd.dtype = s->dtype;
        hd.out_f32 = 1;
        hd.M = NW;
        hd.N = s->vocab;
        hd.K = Wd;
        hd.a = s->hw;
        hd.lda = Wd;
        hd.w = s->head;
        hd.c = s->logits;
        hd.ldc = s->vocab;
        if (launch_stack_gemm(hd, stream))
            return -1;
        if (next_ids_out && launch_argmax(s->ids_out, s->logits, NW, s->vocab, stream))
            return -1;
        if (logits_out)
            HIP_OK(hipMemcpyAsync(logits_out, s->logits, (size_t) NW * s->vocab * 4, hipMemcpyDeviceToHost, stream));
        if (next_ids_out)
            HIP_OK(hipMemcpyAsync(next_ids_out, s->ids_out, (size_t) NW * 4, hipMemcpyDeviceToHost, stream));
    }
    HIP_OK(hipStreamSynchronize(stream));
    return 0;
}

int32_t tllm_stack_page_size(tllm_stack_t s)
{
    return s ? s->page : 0;
}
int32_t tllm_stack_num_blocks(tllm_stack_t s)
{
    return s ? s->blocks : 0;
}
int32_t tllm_stack_num_slots(tllm_stack_t s)
{
    return s ? s->slots : 0;
}
int32_t tllm_stack_vocab(tllm_stack_t s)
{
    return s ? s->vocab : 0;
}
int32_t tllm_stack_layer_runs(tllm_stack_t s)
{
    return s ? (int32_t) s->runs.size() : 0;
}
int64_t tllm_stack_weight_bytes(tllm_stack_t s)
{
    return s ? s->weight_bytes : 0;
}

int64_t tllm_stack_step_bytes(tllm_stack_t s, int32_t n_tokens, int64_t context_tokens, int32_t n_entries)
{
    if (!s)
        return 0;
    // weights once (a looped layer's weights once per pass), keys and values of the contexts once per attention run, states read and
    // written once per recurrent run, the embedding rows instead of the whole table
    int64_t bytes = (int64_t) s->vocab * s->width * s->es + (int64_t) n_tokens * s->width * s->es;
    for (const Run& r : s->runs)
    {
        const Layer& l = s->layers[r.layer];
        bytes += ((int64_t) l.n_mix + l.n_ctx + (l.ff > 0 ? 3 * (int64_t) l.ff + s->width : 0)) * s->width * s->es;
        if (l.kind == MIX_ATTENTION)
            bytes += context_tokens * ((int64_t) l.n_k + l.n_v) * s->es;
        else
            bytes += 2 * (int64_t) n_entries * l.heads * l.dim * l.vdim * 4;
    }
    return bytes;
}

int32_t tllm_stack_get_tap(tllm_stack_t s, int32_t run, float* out, size_t n_floats)
{
    if (!s || !s->taps || !s->tap || run < 0 || run >= (int) s->runs.size() || n_floats != (size_t) s->tap_tokens * s->width)
    {
        set_error("tllm_stack_get_tap: taps are off (debug_taps=1), or run / size do not fit the last step");
        return -1;
    }
    HIP_OK(hipMemcpy(out, s->tap + (size_t) run * s->tap_tokens * s->width, n_floats * 4, hipMemcpyDeviceToHost));
    return 0;
}

void tllm_stack_destroy(tllm_stack_t s)
{
    delete s;
}

} // extern "C"
