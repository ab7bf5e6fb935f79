// The plain scalar decoder as a program, so that it can run under the compiler's address and undefined-behaviour
// checks (a library loaded into Python cannot): reads one case from a file, writes the logits to another.
// File: int32 T, V, H, L, heads, kv_heads, hd, I; float eps; int32 windows[L]; int32 tokens[T];
// float cos[T][hd/2], sin[T][hd/2]; then the weights' floats to the file's end (the order of plain_forward).
#include "plain_scalar.cpp"

#include <cstdio>

int main(int argc, char** argv) {
  if (argc != 3) return 2;
  std::FILE* f = std::fopen(argv[1], "rb");
  if (!f) return 3;
  int32_t dims[8];
  float eps;
  if (std::fread(dims, 4, 8, f) != 8 || std::fread(&eps, 4, 1, f) != 1) return 4;
  const int T = dims[0], V = dims[1], H = dims[2], L = dims[3], heads = dims[4], kv_heads = dims[5], hd = dims[6], I = dims[7];
  std::vector<int32_t> windows(L), tokens(T);
  std::vector<float> cos((size_t)T * (hd / 2)), sin((size_t)T * (hd / 2));
  if (std::fread(windows.data(), 4, L, f) != (size_t)L || std::fread(tokens.data(), 4, T, f) != (size_t)T) return 4;
  if (std::fread(cos.data(), 4, cos.size(), f) != cos.size() || std::fread(sin.data(), 4, sin.size(), f) != sin.size()) return 4;
  const size_t QD = (size_t)heads * hd, KVD = (size_t)kv_heads * hd;
  const size_t need = (size_t)V * H + (size_t)L * (2 * (size_t)H + QD * H + 2 * KVD * H + H * QD + 3 * (size_t)I * H) + H + (size_t)V * H;
  std::vector<float> weights(need);                 // exactly what plain_forward may touch: one float more is an error here
  if (std::fread(weights.data(), 4, need, f) != need) return 5;
  std::fclose(f);
  std::vector<float> logits((size_t)T * V);
  plain_forward(weights.data(), tokens.data(), T, V, H, L, heads, kv_heads, hd, I, eps, windows.data(), cos.data(), sin.data(), logits.data());
  std::FILE* o = std::fopen(argv[2], "wb");
  if (!o || std::fwrite(logits.data(), 4, logits.size(), o) != logits.size()) return 6;
  std::fclose(o);
  return 0;
}
