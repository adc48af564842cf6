// The plain path: the whole model on the host, one element at a time, in formula order, float32 storage
// with float64 accumulation, keys and values in one contiguous run per layer. It is the oracle the engine's
// exact path is held against inside the library itself (the tests carry a second, independent transcription);
// it is read more often than it is run, so nothing is tiled, unrolled or reassociated: a dot product takes its
// terms in ascending k, a norm has its sum of squares before it scales, the softmax normalises once after the
// weighted sum (src/alofa/kernels/cpu/scalar.mojo:1-9; the forward pass src/alofa/model/arch/qwen.mojo:1362-1525).
// Threads only share out independent outputs (columns of a product, heads of the attention); every output's own
// sum is one thread's, in the order above, so results do not depend on the number of threads.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <string>
#include <unordered_map>
#include <vector>

namespace {

constexpr float kLowestF32 = -3.4028234663852886e38f;  // seed of the softmax's maximum (scalar.mojo:32-35)

struct Tensor {
  const float* data = nullptr;
  int64_t count = 0;
};

struct PlainModel {
  int L, h, H, Hkv, d, I, V, max_tokens;
  bool tied;
  float eps;      // kept as float32, widened where used (qwen.mojo:952)
  double theta;
  std::vector<int64_t> window;            // per layer: keys a query sees, 0 for all
  std::unordered_map<std::string, Tensor> tensors;
  std::vector<float> cos_t, sin_t;        // [max_tokens, d]: both halves hold the same values (qwen.mojo:830-880)
  std::vector<std::vector<float>> k_store, v_store;   // per layer [max_tokens, Hkv * d]
  int kv_len = 0;
  std::string error;

  int kv_dim() const { return Hkv * d; }
  const float* need(const std::string& name, int64_t count) {
    auto it = tensors.find(name);
    if (it == tensors.end()) {
      error = "parameter is missing [name=" + name + "]";
      return nullptr;
    }
    if (it->second.count != count) {
      error = "parameter has the wrong size [name=" + name + "]";
      return nullptr;
    }
    return it->second.data;
  }
};

// y = x * 1/sqrt(mean(x^2) + eps) * w: float64 sum in column order, eps inside the root, the weight after the
// scale, one rounding (scalar.mojo:93-129)
void rmsnorm(const float* x, const float* w, float eps, int rows, int cols, float* y) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + static_cast<int64_t>(r) * cols;
    double ss = 0.0;
    for (int c = 0; c < cols; ++c) ss += static_cast<double>(xr[c]) * static_cast<double>(xr[c]);
    const double s = 1.0 / sqrt(ss / cols + static_cast<double>(eps));
    for (int c = 0; c < cols; ++c) y[static_cast<int64_t>(r) * cols + c] = static_cast<float>(static_cast<double>(xr[c]) * s * static_cast<double>(w[c]));
  }
}

// y = x w^T (+ b), w [n_out, n_in] as stored; the accumulator is float64 and starts at the bias (scalar.mojo:132-193)
void linear(const float* x, const float* w, const float* b, int rows, int n_in, int n_out, float* y) {
#pragma omp parallel for schedule(static)
  for (int n = 0; n < n_out; ++n) {
    const float* wn = w + static_cast<int64_t>(n) * n_in;
    for (int m = 0; m < rows; ++m) {
      const float* xm = x + static_cast<int64_t>(m) * n_in;
      double acc = b ? static_cast<double>(b[n]) : 0.0;
      for (int k = 0; k < n_in; ++k) acc += static_cast<double>(xm[k]) * static_cast<double>(wn[k]);
      y[static_cast<int64_t>(m) * n_out + n] = static_cast<float>(acc);
    }
  }
}

// rotate every head's pairs (j, j + d/2) by the row's position, in float32: two products and one sum or
// difference, no fused multiply-add (scalar.mojo:283-344)
void rope(float* x, const PlainModel& m, int rows, int heads, int pos0) {
  const int d = m.d, hf = d / 2;
  for (int r = 0; r < rows; ++r) {
    const float* c = m.cos_t.data() + static_cast<int64_t>(pos0 + r) * d;
    const float* s = m.sin_t.data() + static_cast<int64_t>(pos0 + r) * d;
    for (int hd = 0; hd < heads; ++hd) {
      float* v = x + (static_cast<int64_t>(r) * heads + hd) * d;
      for (int j = 0; j < hf; ++j) {
        const float a = v[j], b = v[j + hf];
        volatile float ac = a * c[j], bs = b * s[j], bc = b * c[j + hf], as = a * s[j + hf];   // (each product rounded by itself)
        v[j] = ac - bs;
        v[j + hf] = bc + as;
      }
    }
  }
}

// causal grouped-query attention of `rows` queries, the first at position pos0, over the layer's store: the dot
// in float64 rounded to float32, times float32 1/sqrt(float32 d); maximum and exp in float32; the weights' sum and
// the weighted sum of values in float64, one division per channel at the end (scalar.mojo:392-470)
void attention(const float* q, const std::vector<float>& ks, const std::vector<float>& vs, const PlainModel& m, int rows, int pos0,
               int64_t window, float* out) {
  const int d = m.d, g = m.H / m.Hkv, kv = m.kv_dim();
  const float scale = 1.0f / sqrtf(static_cast<float>(d));
#pragma omp parallel for schedule(dynamic) collapse(2)
  for (int r = 0; r < rows; ++r) {
    for (int hq = 0; hq < m.H; ++hq) {
      const int hk = hq / g, pos = pos0 + r;
      const int first = window > 0 && pos - window + 1 > 0 ? static_cast<int>(pos - window + 1) : 0;
      const float* qv = q + (static_cast<int64_t>(r) * m.H + hq) * d;
      std::vector<float> s(pos - first + 1);
      float big = kLowestF32;
      for (int j = first; j <= pos; ++j) {
        const float* kj = ks.data() + static_cast<int64_t>(j) * kv + hk * d;
        double dot = 0.0;
        for (int c = 0; c < d; ++c) dot += static_cast<double>(qv[c]) * static_cast<double>(kj[c]);
        const float sj = static_cast<float>(dot) * scale;
        s[j - first] = sj;
        if (sj > big) big = sj;
      }
      double z = 0.0;
      for (int j = first; j <= pos; ++j) {
        const float e = expf(s[j - first] - big);
        s[j - first] = e;
        z += static_cast<double>(e);
      }
      for (int c = 0; c < d; ++c) {
        double acc = 0.0;
        for (int j = first; j <= pos; ++j) acc += static_cast<double>(s[j - first]) * static_cast<double>(vs[static_cast<int64_t>(j) * kv + hk * d + c]);
        out[(static_cast<int64_t>(r) * m.H + hq) * d + c] = static_cast<float>(acc / z);
      }
    }
  }
}

thread_local std::string g_plain_error;

int fail(const std::string& text) {
  g_plain_error = text;
  return -1;
}

}  // namespace

extern "C" {

const char* alofa_plain_last_error() { return g_plain_error.c_str(); }

// sizes: layers, hidden, heads, kv_heads, head_dim, intermediate, vocab, tied (0/1), max_tokens; windows: per layer, 0 for none
void* alofa_plain_new(const int64_t* sizes, double eps, double theta, const int64_t* windows) {
  PlainModel* m = new PlainModel();
  m->L = static_cast<int>(sizes[0]), m->h = static_cast<int>(sizes[1]), m->H = static_cast<int>(sizes[2]), m->Hkv = static_cast<int>(sizes[3]);
  m->d = static_cast<int>(sizes[4]), m->I = static_cast<int>(sizes[5]), m->V = static_cast<int>(sizes[6]), m->tied = sizes[7] != 0;
  m->max_tokens = static_cast<int>(sizes[8]);
  m->eps = static_cast<float>(eps), m->theta = theta;
  if (m->L <= 0 || m->h <= 0 || m->H <= 0 || m->Hkv <= 0 || m->H % m->Hkv || m->d <= 0 || m->d % 2 || m->I <= 0 || m->V <= 0 || m->max_tokens <= 0) {
    delete m;
    fail("sizes must be positive, kv_heads divide heads, head_dim be even");
    return nullptr;
  }
  m->window.assign(windows, windows + m->L);
  // the table as the reference builds it: the inverse frequency and the angle in float32, cos and sin evaluated in
  // float64 and rounded once (qwen.mojo:830-880)
  const int d = m->d, hf = d / 2;
  m->cos_t.resize(static_cast<size_t>(m->max_tokens) * d), m->sin_t.resize(static_cast<size_t>(m->max_tokens) * d);
  for (int p = 0; p < m->max_tokens; ++p)
    for (int i = 0; i < hf; ++i) {
      const float inv = 1.0f / static_cast<float>(pow(m->theta, static_cast<double>(2 * i) / static_cast<double>(d)));
      volatile float ang = static_cast<float>(p) * inv;
      const float c = static_cast<float>(cos(static_cast<double>(ang))), s = static_cast<float>(sin(static_cast<double>(ang)));
      m->cos_t[static_cast<size_t>(p) * d + i] = m->cos_t[static_cast<size_t>(p) * d + i + hf] = c;
      m->sin_t[static_cast<size_t>(p) * d + i] = m->sin_t[static_cast<size_t>(p) * d + i + hf] = s;
    }
  m->k_store.assign(m->L, std::vector<float>(static_cast<size_t>(m->max_tokens) * m->kv_dim()));
  m->v_store.assign(m->L, std::vector<float>(static_cast<size_t>(m->max_tokens) * m->kv_dim()));
  return m;
}
void alofa_plain_free(void* m) { delete static_cast<PlainModel*>(m); }

// The tensor's float32 values stay the caller's: they must outlive the model.
int alofa_plain_set_tensor(void* mv, const char* name, const float* data, int64_t count) {
  static_cast<PlainModel*>(mv)->tensors[name] = Tensor{data, count};
  return 0;
}
void alofa_plain_reset(void* mv) { static_cast<PlainModel*>(mv)->kv_len = 0; }
int alofa_plain_length(void* mv) { return static_cast<PlainModel*>(mv)->kv_len; }

// The forward pass over `n` new tokens that extend the stored history. logits: float [n, vocab] when all_rows,
// else [1, vocab] for the last row only, as the reference (qwen.mojo:1512-1525).
int alofa_plain_run(void* mv, const int* ids, int n, int all_rows, float* logits) {
  PlainModel& m = *static_cast<PlainModel*>(mv);
  if (n <= 0) return fail("no tokens given");
  const int pos0 = m.kv_len;
  if (pos0 + n > m.max_tokens) return fail("history would exceed the allocated length [kv_len=" + std::to_string(pos0 + n) + " max=" + std::to_string(m.max_tokens) + "]");
  const int h = m.h, kv = m.kv_dim(), qd = m.H * m.d;
  const float* embed = m.need("model.embed_tokens.weight", static_cast<int64_t>(m.V) * h);
  if (!embed) return fail(m.error);
  std::vector<float> hidden(static_cast<size_t>(n) * h), normed(static_cast<size_t>(n) * h), q(static_cast<size_t>(n) * qd), k(static_cast<size_t>(n) * kv),
      v(static_cast<size_t>(n) * kv), attn(static_cast<size_t>(n) * qd), proj(static_cast<size_t>(n) * h), gate(static_cast<size_t>(n) * m.I), up(static_cast<size_t>(n) * m.I);
  for (int i = 0; i < n; ++i) {
    if (ids[i] < 0 || ids[i] >= m.V) return fail("token id is outside the vocabulary [id=" + std::to_string(ids[i]) + "]");
    memcpy(hidden.data() + static_cast<size_t>(i) * h, embed + static_cast<size_t>(ids[i]) * h, sizeof(float) * h);   // no scaling (qwen.mojo:1391-1413)
  }
  for (int layer = 0; layer < m.L; ++layer) {
    const std::string p = "model.layers." + std::to_string(layer) + ".";
    const float* w_in = m.need(p + "input_layernorm.weight", h);
    const float* wq = m.need(p + "self_attn.q_proj.weight", static_cast<int64_t>(qd) * h);
    const float* bq = m.need(p + "self_attn.q_proj.bias", qd);
    const float* wk = m.need(p + "self_attn.k_proj.weight", static_cast<int64_t>(kv) * h);
    const float* bk = m.need(p + "self_attn.k_proj.bias", kv);
    const float* wv = m.need(p + "self_attn.v_proj.weight", static_cast<int64_t>(kv) * h);
    const float* bv = m.need(p + "self_attn.v_proj.bias", kv);
    const float* wo = m.need(p + "self_attn.o_proj.weight", static_cast<int64_t>(h) * qd);
    const float* w_post = m.need(p + "post_attention_layernorm.weight", h);
    const float* wg = m.need(p + "mlp.gate_proj.weight", static_cast<int64_t>(m.I) * h);
    const float* wu = m.need(p + "mlp.up_proj.weight", static_cast<int64_t>(m.I) * h);
    const float* wd = m.need(p + "mlp.down_proj.weight", static_cast<int64_t>(h) * m.I);
    if (!w_in || !wq || !bq || !wk || !bk || !wv || !bv || !wo || !w_post || !wg || !wu || !wd) return fail(m.error);
    // input norm; q, k, v with bias; rotate q and k, not v; append to the store; attend over the whole store;
    // output projection without bias; residual sum in float32 (qwen.mojo:1418-1480)
    rmsnorm(hidden.data(), w_in, m.eps, n, h, normed.data());
    linear(normed.data(), wq, bq, n, h, qd, q.data());
    linear(normed.data(), wk, bk, n, h, kv, k.data());
    linear(normed.data(), wv, bv, n, h, kv, v.data());
    rope(q.data(), m, n, m.H, pos0);
    rope(k.data(), m, n, m.Hkv, pos0);
    memcpy(m.k_store[layer].data() + static_cast<size_t>(pos0) * kv, k.data(), sizeof(float) * n * kv);
    memcpy(m.v_store[layer].data() + static_cast<size_t>(pos0) * kv, v.data(), sizeof(float) * n * kv);
    attention(q.data(), m.k_store[layer], m.v_store[layer], m, n, pos0, m.window[layer], attn.data());
    linear(attn.data(), wo, nullptr, n, qd, h, proj.data());
    for (size_t i = 0; i < hidden.size(); ++i) hidden[i] = hidden[i] + proj[i];
    // feed-forward norm; gate and up without bias; silu(gate) * up with the sigmoid's exp in float64; down
    // projection; residual sum (scalar.mojo:219-231; qwen.mojo:1482-1510)
    rmsnorm(hidden.data(), w_post, m.eps, n, h, normed.data());
    linear(normed.data(), wg, nullptr, n, h, m.I, gate.data());
    linear(normed.data(), wu, nullptr, n, h, m.I, up.data());
    for (size_t i = 0; i < gate.size(); ++i) {
      const double g = static_cast<double>(gate[i]);
      gate[i] = static_cast<float>(g / (1.0 + exp(-g)) * static_cast<double>(up[i]));
    }
    linear(gate.data(), wd, nullptr, n, m.I, h, proj.data());
    for (size_t i = 0; i < hidden.size(); ++i) hidden[i] = hidden[i] + proj[i];
  }
  m.kv_len = pos0 + n;
  // final norm and the output matrix on the wanted rows: the head's own matrix if the file has it, else the
  // embedding when tied, else an error (qwen.mojo:1080-1089)
  const float* w_norm = m.need("model.norm.weight", h);
  if (!w_norm) return fail(m.error);
  const float* head = m.tensors.count("lm_head.weight") ? m.need("lm_head.weight", static_cast<int64_t>(m.V) * h) : (m.tied ? embed : nullptr);
  if (!head) return fail(m.tensors.count("lm_head.weight") ? m.error : "no output matrix: lm_head.weight is absent and the embedding is not tied");
  const int first = all_rows ? 0 : n - 1, rows = n - first;
  rmsnorm(hidden.data() + static_cast<size_t>(first) * h, w_norm, m.eps, rows, h, normed.data());
  linear(normed.data(), head, nullptr, rows, h, m.V, logits);
  return rows;
}

// the first maximum: strict >, the lowest index wins ties (qwen.mojo:1527-1541)
int alofa_plain_argmax(const float* row, int n) {
  float best = kLowestF32;
  int at = 0;
  for (int i = 0; i < n; ++i)
    if (row[i] > best) best = row[i], at = i;
  return at;
}

}  // extern "C"
