// Kernels of the routed feed-forward (a mixture of gated experts).
//   * route: per token the router's logits (32-bit, from 32-bit router weights), their softmax over
//     all experts, the choice of `top` experts by score + correction, restricted to the best `keep`
//     of `groups` equal groups of neighbouring experts (a group's score is its best corrected
//     score), and the chosen experts' softmax scores divided by their sum.  The result is a dense
//     row of weights per token, zero where an expert was not chosen.  Optionally the sigmoid gate
//     of an expert that every token uses (one number per token).
//   * gated activation: hidden = weight * silu(gate) * up for every expert side by side (and the
//     always-on expert with its sigmoid gate as weight), so that ONE product with the experts' down
//     matrices laid side by side gives the weighted sum of their outputs; experts whose output is
//     their input ("identity experts", the last router outputs) leave weight * h as 32-bit rows.
// Ties between equal scores go to the lower index.
#include "host.h"

#define ROUTE_THREADS 256
#define ROUTE_MAX_EXPERTS 1024

struct RouteCall {
  int dtype;                // element type of `h`: 0 float32, 1 bfloat16
  int tokens, width;
  int experts;              // router outputs: experts with tensors and identity experts together
  int top;
  int groups, keep;         // groups <= 1: every expert can be chosen
  const void* h;            // [tokens][ldh]
  int64_t ldh;
  const float* W;           // [experts][width] float32
  const float* correction;  // [experts] or null: added to the scores for the choice only
  const float* gate_w;      // [width] float32 or null
  float* weights;           // [tokens][experts]
  float* gate;              // [tokens]: sigmoid(gate_w . h), or null
};

template <typename T>
__global__ void __launch_bounds__(ROUTE_THREADS) route_kernel(RouteCall c) {
  extern __shared__ float hrow[];                 // [width]
  __shared__ float score[ROUTE_MAX_EXPERTS];      // logits, then softmax scores
  __shared__ float choice[ROUTE_MAX_EXPERTS];     // scores with the correction; -inf once taken or shut out
  __shared__ float scratch[32];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = ROUTE_THREADS / 64;
  const T* h = static_cast<const T*>(c.h) + (int64_t)t * c.ldh;
  for (int col = threadIdx.x; col < c.width; col += ROUTE_THREADS) hrow[col] = to_float(h[col]);
  __syncthreads();
  const int outputs = c.experts + (c.gate_w ? 1 : 0);
  for (int e = wave; e < outputs; e += waves) {
    const float* w = e < c.experts ? c.W + (int64_t)e * c.width : c.gate_w;
    float sum = 0.f;
    for (int col = lane; col < c.width; col += 64) sum = fmaf(w[col], hrow[col], sum);
    sum = wave_sum(sum);
    if (lane == 0) {
      if (e < c.experts) score[e] = sum;
      else c.gate[t] = 1.0f / (1.0f + expf(-sum));
    }
  }
  __syncthreads();
  float top_logit = -INFINITY;
  for (int e = threadIdx.x; e < c.experts; e += ROUTE_THREADS) top_logit = fmaxf(top_logit, score[e]);
  top_logit = block_max(top_logit, scratch);
  float total = 0.f;
  for (int e = threadIdx.x; e < c.experts; e += ROUTE_THREADS) total += expf(score[e] - top_logit);
  total = block_sum(total, scratch);
  __syncthreads();
  for (int e = threadIdx.x; e < c.experts; e += ROUTE_THREADS) {
    const float s = expf(score[e] - top_logit) / total;
    score[e] = s;
    choice[e] = s + (c.correction ? c.correction[e] : 0.f);
    c.weights[(int64_t)t * c.experts + e] = 0.f;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  // the choice itself is short and serial: a few hundred comparisons
  if (c.groups > 1) {
    // a group's score is its best corrected score; the best `keep` groups stay open, the experts of
    // the others are shut out (minus infinity, since corrected scores may be negative)
    const int per = c.experts / c.groups;
    unsigned long long open = 0ull;
    for (int kept = 0; kept < c.keep; ++kept) {
      int best = -1;
      float best_score = -INFINITY;
      for (int g = 0; g < c.groups; ++g) {
        if ((open >> g) & 1ull) continue;
        float group_score = -INFINITY;
        for (int i = 0; i < per; ++i) group_score = fmaxf(group_score, choice[g * per + i]);
        if (best < 0 || group_score > best_score) { best = g; best_score = group_score; }
      }
      open |= 1ull << best;
    }
    for (int g = 0; g < c.groups; ++g)
      if (!((open >> g) & 1ull))
        for (int i = 0; i < per; ++i) choice[g * per + i] = -INFINITY;
  }
  float sum = 0.f;
  int chosen[64];
  const int top = c.top < 64 ? c.top : 64;
  for (int k = 0; k < top; ++k) {
    int best = 0;
    float best_score = choice[0];
    for (int e = 1; e < c.experts; ++e)
      if (choice[e] > best_score) { best = e; best_score = choice[e]; }
    chosen[k] = best;
    choice[best] = -INFINITY;
    sum += score[best];
  }
  const float inverse = 1.0f / (sum + 1e-20f);
  for (int k = 0; k < top; ++k) c.weights[(int64_t)t * c.experts + chosen[k]] = score[chosen[k]] * inverse;
}

BT_EXPORT int bt_route_call(void* stream, const RouteCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->experts <= 0 || c->experts > ROUTE_MAX_EXPERTS) BT_REFUSE("route: %d experts outside 1..%d", c->experts, ROUTE_MAX_EXPERTS);
  if (c->top <= 0 || c->top > c->experts || c->top > 64) BT_REFUSE("route: %d of %d experts a token (at most 64)", c->top, c->experts);
  if (c->groups > 1) {
    if (c->groups > 64 || c->experts % c->groups != 0 || c->keep <= 0 || c->keep > c->groups)
      BT_REFUSE("route: %d groups (at most 64) must divide %d experts, and 1..groups of them stay open, not %d", c->groups, c->experts, c->keep);
    if (c->keep * (c->experts / c->groups) < c->top)
      BT_REFUSE("route: %d open groups of %d experts cannot give %d experts", c->keep, c->experts / c->groups, c->top);
  }
  if (c->width <= 0 || c->width > 15360) BT_REFUSE("route: width %d outside 1..15360", c->width);
  if (!c->h || !c->W || !c->weights || (c->gate_w && !c->gate)) BT_REFUSE("route: missing operand");
  dim3 grid(c->tokens), block(ROUTE_THREADS);
  const size_t lds = (size_t)c->width * sizeof(float);
  if (c->dtype == 0)
    hipLaunchKernelGGL(route_kernel<float>, grid, block, lds, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(route_kernel<bf16_t>, grid, block, lds, (hipStream_t)stream, *c);
  return bt_check_launch("route");
}

struct GatedExpertsCall {
  int dtype;                // element type of `gu`, `hidden` and `h`
  int tokens;
  int experts;              // experts with tensors, each `ff` wide
  int ff;
  int shared_ff;            // width of the expert every token uses; 0: none
  int identity;             // identity experts: router outputs experts .. experts + identity - 1
  int hidden_cols;          // columns of `hidden` written: experts * ff + shared_ff, then zeros
  int width;
  const void* gu;           // [tokens][ld_gu]: per expert its gate rows (ff) then its up rows (ff); then the shared expert's
  int64_t ld_gu;
  const float* weights;     // [tokens][experts + identity]
  const float* gate;        // [tokens]: the shared expert's weight, or null
  void* hidden;             // [tokens][ld_hidden]
  int64_t ld_hidden;
  const void* h;            // [tokens][ldh]: the experts' input (read for identity experts only)
  int64_t ldh;
  float* identity_out;      // [tokens][width] float32: (sum of the identity experts' weights) * h; or null
};

template <typename T>
__global__ void __launch_bounds__(256) gated_experts_kernel(GatedExpertsCall c) {
  const int t = blockIdx.x;
  const T* gu = static_cast<const T*>(c.gu) + (int64_t)t * c.ld_gu;
  T* hidden = static_cast<T*>(c.hidden) + (int64_t)t * c.ld_hidden;
  const float* weights = c.weights + (int64_t)t * (c.experts + c.identity);
  const int routed = c.experts * c.ff;
  for (int col = threadIdx.x; col < c.hidden_cols; col += blockDim.x) {
    float out = 0.f;
    if (col < routed) {
      const int e = col / c.ff, i = col - e * c.ff;
      const float w = weights[e];
      if (w != 0.f) {
        const float g = to_float(gu[(int64_t)e * 2 * c.ff + i]), u = to_float(gu[(int64_t)e * 2 * c.ff + c.ff + i]);
        out = w * (g / (1.0f + expf(-g))) * u;
      }
    } else if (col < routed + c.shared_ff) {
      const int i = col - routed;
      const float g = to_float(gu[(int64_t)2 * routed + i]), u = to_float(gu[(int64_t)2 * routed + c.shared_ff + i]);
      out = (c.gate ? c.gate[t] : 1.0f) * (g / (1.0f + expf(-g))) * u;
    }
    hidden[col] = from_float<T>(out);
  }
  if (c.identity_out) {
    float w = 0.f;
    for (int i = 0; i < c.identity; ++i) w += weights[c.experts + i];
    const T* h = static_cast<const T*>(c.h) + (int64_t)t * c.ldh;
    for (int col = threadIdx.x; col < c.width; col += blockDim.x)
      c.identity_out[(int64_t)t * c.width + col] = w != 0.f ? w * to_float(h[col]) : 0.f;
  }
}

BT_EXPORT int bt_gated_experts_call(void* stream, const GatedExpertsCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->experts < 0 || c->ff <= 0 || c->shared_ff < 0 || c->identity < 0)
    BT_REFUSE("gated_experts: %d experts of %d, a shared one of %d and %d identity experts", c->experts, c->ff, c->shared_ff, c->identity);
  const int64_t columns = (int64_t)c->experts * c->ff + c->shared_ff;
  if (c->hidden_cols < columns || c->ld_hidden < c->hidden_cols || c->ld_gu < 2 * columns)
    BT_REFUSE("gated_experts: the rows do not hold the experts");
  if (!c->gu || !c->weights || !c->hidden || (c->identity_out && (!c->h || c->width <= 0)))
    BT_REFUSE("gated_experts: missing operand");
  dim3 grid(c->tokens), block(256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(gated_experts_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(gated_experts_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("gated_experts");
}
