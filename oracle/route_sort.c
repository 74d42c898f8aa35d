/* CPU oracle, plain C. TEST INFRASTRUCTURE ONLY: never linked into the product library.
 *
 * A second, independent restatement of the integer parts of the OLMoE MoE layer, written
 * the way the reference's native file walks them (paths under the reference tree):
 *
 *   oracle_route           switchyard/csrc/moe_kernels.cu:23-71  (softmax in fp32, k rounds of
 *                          arg-max, ties to the lower expert id; weight = p or p / sum of k)
 *   oracle_sort_by_expert  switchyard/csrc/moe_kernels.cu:112-157 (for each expert walk the
 *                          flat choices in order; counts, offsets, token, wsorted, pos_of)
 *   oracle_combine_order   switchyard/csrc/moe_kernels.cu:422-427 (a token's k slots ordered
 *                          by expert id, stable)
 *   oracle_experts_f32     switchyard/moe.py:34-42 in scalar fp32 (small shapes only)
 *
 * The selection key is the logit itself, not exp(logit - max): exp is monotone, so the two
 * agree wherever exp keeps distinct logits distinct, and the logit key is exact everywhere.
 *
 * Pinned by tests/test_oracle.py against the reference's known-answer test for the sort
 * (tests/test_model.py:49-57) and against the torch restatement in oracle/moe_oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

int oracle_route(const float* logits, int N, int E, int k, int norm, int32_t* idx, float* w) {
  if (k > E || k > 64) return 1;
  unsigned char* taken = (unsigned char*)malloc((size_t)E);
  if (!taken) return 2;
  for (int t = 0; t < N; ++t) {
    const float* row = logits + (size_t)t * E;
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) mx = row[e] > mx ? row[e] : mx;
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(row[e] - mx);
    memset(taken, 0, (size_t)E);
    float total = 0.f, picked[64];
    for (int r = 0; r < k; ++r) {
      int be = -1;
      for (int e = 0; e < E; ++e)
        if (!taken[e] && (be < 0 || row[e] > row[be])) be = e; /* strict >: lower id wins ties */
      taken[be] = 1;
      idx[(size_t)t * k + r] = be;
      picked[r] = expf(row[be] - mx) / sum;
      total += picked[r];
    }
    for (int r = 0; r < k; ++r) w[(size_t)t * k + r] = norm ? picked[r] / total : picked[r];
  }
  free(taken);
  return 0;
}

/* w is carried as opaque 16-bit or 32-bit words (wbytes = 2 or 4): a pure permutation. */
int oracle_sort_by_expert(const int32_t* idx, const void* w, int wbytes, int M, int k, int E,
                          int32_t* counts, int32_t* offsets, int32_t* token, void* wsorted,
                          int32_t* pos_of) {
  if (wbytes != 2 && wbytes != 4) return 1;
  for (int e = 0; e < E; ++e) {
    int n = 0;
    for (int i = 0; i < M; ++i) n += idx[i] == e;
    counts[e] = n;
  }
  offsets[0] = 0;
  for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
  for (int e = 0; e < E; ++e) {
    int at = offsets[e];
    for (int i = 0; i < M; ++i) {
      if (idx[i] != e) continue;
      token[at] = i / k;
      memcpy((char*)wsorted + (size_t)at * wbytes, (const char*)w + (size_t)i * wbytes, (size_t)wbytes);
      pos_of[i] = at;
      ++at;
    }
  }
  return 0;
}

/* order[t*k + j] = the slot holding token t's j-th smallest expert id (stable). */
void oracle_combine_order(const int32_t* idx, int N, int k, int32_t* order) {
  for (int t = 0; t < N; ++t) {
    int32_t* o = order + (size_t)t * k;
    const int32_t* id = idx + (size_t)t * k;
    for (int j = 0; j < k; ++j) o[j] = j;
    for (int a = 1; a < k; ++a)
      for (int b = a; b > 0 && id[o[b]] < id[o[b - 1]]; --b) {
        int32_t x = o[b]; o[b] = o[b - 1]; o[b - 1] = x;
      }
  }
}

/* out[N,H] = sum over experts ascending of w * down[e] @ (silu(gate[e] @ h) * (up[e] @ h)),
 * scalar fp32, products accumulated left to right. gate_up [E,2I,H], down [E,H,I]. */
int oracle_experts_f32(const float* h, const int32_t* idx, const float* w, const float* gate_up,
                       const float* down, int N, int k, int E, int H, int I, float* out) {
  float* act = (float*)malloc(sizeof(float) * (size_t)I);
  if (!act) return 2;
  memset(out, 0, sizeof(float) * (size_t)N * H);
  for (int e = 0; e < E; ++e) {
    const float* gu = gate_up + (size_t)e * 2 * I * H;
    const float* dn = down + (size_t)e * H * I;
    for (int t = 0; t < N; ++t)
      for (int s = 0; s < k; ++s) {
        if (idx[(size_t)t * k + s] != e) continue;
        const float* x = h + (size_t)t * H;
        for (int i = 0; i < I; ++i) {
          float g = 0.f, u = 0.f;
          for (int j = 0; j < H; ++j) {
            g += gu[(size_t)i * H + j] * x[j];
            u += gu[(size_t)(I + i) * H + j] * x[j];
          }
          act[i] = g / (1.f + expf(-g)) * u;
        }
        for (int j = 0; j < H; ++j) {
          float y = 0.f;
          for (int i = 0; i < I; ++i) y += dn[(size_t)j * I + i] * act[i];
          out[(size_t)t * H + j] += y * w[(size_t)t * k + s];
        }
      }
  }
  free(act);
  return 0;
}
