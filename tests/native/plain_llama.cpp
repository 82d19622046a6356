// A second plain implementation of the Llama 3 forward pass, in C++ and in another form than tests/plain.py:
// token by token with a growing list of keys and values (the recurrent form a decoder runs), float64 throughout,
// scalar loops only.  It shares nothing with tests/plain.py, with the engine or with its kernels; the two plain
// implementations are compared with each other (tests/test_plain_second.py), and the engine with the first.
//
// Formulas, from the reference:
//   embedding row, no scaling                      /root/reference/engine/src/model.rs:672-684
//   rmsnorm: x * w / sqrt(mean(x^2) + eps)         /root/reference/kernels/src/ggml/ops_llama.rs:201-216
//   q, k, v = W x (no bias); rope on q and k, split-half pairs (d, d + D/2), angle = pos * inv_freq[d]
//                                                  /root/reference/kernels/src/rope.rs:18-53
//   inv_freq and the llama3 rule on wavelengths    /root/reference/kernels/src/rope.rs:36,848-881
//   scores = q . k / sqrt(D) over keys 0..pos (or the last `window`), softmax, sum p v; kv head = head / (nH / nKV)
//                                                  /root/reference/kernels/src/attention.rs:28-87, model.rs:1078
//   h += Wo a; h += Wdown (silu(Wgate x) * Wup x), x = rmsnorm(h)   /root/reference/engine/src/model.rs:952-1314
//   silu(x) = x / (1 + exp(-x))                    /root/reference/kernels/src/ggml/vec_llama.rs:808-810
//   logits = Whead rmsnorm(h), Whead = embedding when tied          /root/reference/engine/src/model.rs:1355-1398
//
// usage: plain_llama IN OUT.  IN (little endian): int32 {magic 0x4c4c414d, hidden, intermediate, layers, heads,
// kv_heads, head_dim, vocab, tied, n_tokens, window}; int32 windowed[layers]; float64 {eps, theta, scaled, factor,
// low_freq_factor, high_freq_factor, original_max_position}; int32 tokens[n_tokens]; then float64 tensors:
// embedding [vocab, hidden]; per layer input norm [hidden], q [heads * head_dim, hidden], k, v [kv_heads * head_dim,
// hidden], o [hidden, heads * head_dim], post-attention norm [hidden], gate, up [intermediate, hidden], down [hidden,
// intermediate]; final norm [hidden]; head [vocab, hidden] unless tied.  OUT: float64 logits [n_tokens, vocab].
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

typedef std::vector<double> vec;

static void need(bool ok, const char* what) {
  if (!ok) {
    fprintf(stderr, "plain_llama: %s\n", what);
    exit(2);
  }
}

static vec read_doubles(FILE* f, size_t n) {
  vec v(n);
  need(fread(v.data(), sizeof(double), n, f) == n, "input ends early");
  return v;
}

// y = W x, W [rows, cols] row-major
static vec matvec(const vec& W, const vec& x, int rows, int cols) {
  vec y(rows, 0.0);
  for (int r = 0; r < rows; ++r) {
    double acc = 0.0;
    const double* w = &W[(size_t)r * cols];
    for (int c = 0; c < cols; ++c) acc += w[c] * x[c];
    y[r] = acc;
  }
  return y;
}

static vec rmsnorm(const vec& x, const vec& w, double eps) {
  double ss = 0.0;
  for (double v : x) ss += v * v;
  const double inv = 1.0 / sqrt(ss / (double)x.size() + eps);
  vec y(x.size());
  for (size_t i = 0; i < x.size(); ++i) y[i] = x[i] * inv * w[i];
  return y;
}

struct Layer {
  vec in_norm, wq, wk, wv, wo, post_norm, gate, up, down;
  std::vector<vec> keys, values;   // one entry per position: [kv_heads * head_dim]
};

int main(int argc, char** argv) {
  need(argc == 3, "usage: plain_llama IN OUT");
  FILE* f = fopen(argv[1], "rb");
  need(f != nullptr, "cannot open the input");
  int32_t hd[11];
  need(fread(hd, 4, 11, f) == 11 && hd[0] == 0x4c4c414d, "bad header");
  const int H = hd[1], I = hd[2], L = hd[3], nH = hd[4], nKV = hd[5], D = hd[6], V = hd[7], tied = hd[8], T = hd[9], window = hd[10];
  std::vector<int32_t> windowed(L);
  need(fread(windowed.data(), 4, L, f) == (size_t)L, "input ends early");
  double c[7];
  need(fread(c, 8, 7, f) == 7, "input ends early");
  const double eps = c[0], theta = c[1];
  std::vector<int32_t> tokens(T);
  need(fread(tokens.data(), 4, T, f) == (size_t)T, "input ends early");
  const vec embed = read_doubles(f, (size_t)V * H);
  std::vector<Layer> layers(L);
  for (Layer& l : layers) {
    l.in_norm = read_doubles(f, H);
    l.wq = read_doubles(f, (size_t)nH * D * H);
    l.wk = read_doubles(f, (size_t)nKV * D * H);
    l.wv = read_doubles(f, (size_t)nKV * D * H);
    l.wo = read_doubles(f, (size_t)H * nH * D);
    l.post_norm = read_doubles(f, H);
    l.gate = read_doubles(f, (size_t)I * H);
    l.up = read_doubles(f, (size_t)I * H);
    l.down = read_doubles(f, (size_t)H * I);
  }
  const vec final_norm = read_doubles(f, H);
  vec head_own;
  if (!tied) head_own = read_doubles(f, (size_t)V * H);
  const vec& head = tied ? embed : head_own;
  fclose(f);

  // rotation frequencies
  const int half = D / 2;
  vec inv_freq(half);
  const double two_pi = 6.283185307179586476925286766559;
  for (int d = 0; d < half; ++d) {
    double freq = 1.0 / pow(theta, 2.0 * d / (double)D);
    if (c[2] != 0.0) {
      const double factor = c[3], low = c[4], high = c[5], orig = c[6];
      const double wavelen = two_pi / freq;
      if (wavelen < orig / high) {
        // short waves turn as they are
      } else if (wavelen > orig / low) {
        freq /= factor;
      } else {
        const double smooth = (orig / wavelen - low) / (high - low);
        freq = (1.0 - smooth) * freq / factor + smooth * freq;
      }
    }
    inv_freq[d] = freq;
  }
  auto rotate = [&](vec& x, int heads, int pos) {
    for (int h = 0; h < heads; ++h)
      for (int d = 0; d < half; ++d) {
        const double a = (double)pos * inv_freq[d], cs = cos(a), sn = sin(a);
        double& x0 = x[(size_t)h * D + d];
        double& x1 = x[(size_t)h * D + d + half];
        const double r0 = x0 * cs - x1 * sn, r1 = x0 * sn + x1 * cs;
        x0 = r0;
        x1 = r1;
      }
  };

  FILE* out = fopen(argv[2], "wb");
  need(out != nullptr, "cannot open the output");
  const int group = nH / nKV;
  const double scale = 1.0 / sqrt((double)D);
  for (int pos = 0; pos < T; ++pos) {
    need(tokens[pos] >= 0 && tokens[pos] < V, "token outside the vocabulary");
    vec h(embed.begin() + (size_t)tokens[pos] * H, embed.begin() + (size_t)(tokens[pos] + 1) * H);
    for (int li = 0; li < L; ++li) {
      Layer& l = layers[li];
      vec x = rmsnorm(h, l.in_norm, eps);
      vec q = matvec(l.wq, x, nH * D, H), k = matvec(l.wk, x, nKV * D, H), v = matvec(l.wv, x, nKV * D, H);
      rotate(q, nH, pos);
      rotate(k, nKV, pos);
      l.keys.push_back(k);
      l.values.push_back(v);
      int first = 0;
      if (window > 0 && windowed[li] && pos >= window) first = pos - window + 1;
      vec a((size_t)nH * D, 0.0);
      for (int hh = 0; hh < nH; ++hh) {
        const int kvh = hh / group;
        vec s(pos - first + 1);
        double mx = -INFINITY;
        for (int j = first; j <= pos; ++j) {
          double dot = 0.0;
          for (int d = 0; d < D; ++d) dot += q[(size_t)hh * D + d] * l.keys[j][(size_t)kvh * D + d];
          s[j - first] = dot * scale;
          mx = fmax(mx, s[j - first]);
        }
        double sum = 0.0;
        for (double& e : s) {
          e = exp(e - mx);
          sum += e;
        }
        for (int j = first; j <= pos; ++j) {
          const double p = s[j - first] / sum;
          for (int d = 0; d < D; ++d) a[(size_t)hh * D + d] += p * l.values[j][(size_t)kvh * D + d];
        }
      }
      const vec o = matvec(l.wo, a, H, nH * D);
      for (int i = 0; i < H; ++i) h[i] += o[i];
      x = rmsnorm(h, l.post_norm, eps);
      const vec g = matvec(l.gate, x, I, H), u = matvec(l.up, x, I, H);
      vec act(I);
      for (int i = 0; i < I; ++i) act[i] = g[i] / (1.0 + exp(-g[i])) * u[i];
      const vec dn = matvec(l.down, act, H, I);
      for (int i = 0; i < H; ++i) h[i] += dn[i];
    }
    const vec logits = matvec(head, rmsnorm(h, final_norm, eps), V, H);
    need(fwrite(logits.data(), 8, V, out) == (size_t)V, "cannot write");
  }
  fclose(out);
  return 0;
}
