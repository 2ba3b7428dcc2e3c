// Fused multi-tensor Adam step: the optimizer the reference trains every parameter group with,
// torch.optim.Adam(lr=0.0, eps=1e-15) with per-group learning rates (scene/gaussian_model.py:574;
// stepped at train_internal.py:404-417, after "param.grad /= bsz" at :407-410, which is folded in here as
// grad_scale).  Update rule of torch 2.0.0 (the version the reference pins), default betas, no weight
// decay, no amsgrad:
// (hyper-parameters arrive as doubles, like the Python floats of that optimizer: 1-b is formed in double
// and only then rounded to fp32)
//   m = m*b1 + (1-b1)*g;  v = v*b2 + (1-b2)*g*g;
//   p = p - (lr / (1-b1^t)) * m / (sqrt(v)/sqrt(1-b2^t) + eps)
// One launch covers up to ADAM_MAX_TENSORS tensors: a workgroup looks its (tensor, chunk) up in a small
// table passed by value, so the ~20 small MLP tensors cost no launches of their own.  28 bytes per
// element (p, g, m, v in; p, m, v out), 16-byte accesses wherever the four pointers allow.
#include "gs_common.h"
#include "gs_kernels.h"

namespace gs {

namespace {

constexpr int ADAM_THREADS = 256;
constexpr int ADAM_VEC = 4;
constexpr int ADAM_ITEMS = 4;  // 16-byte vectors per thread
constexpr int ADAM_CHUNK = ADAM_THREADS * ADAM_VEC * ADAM_ITEMS;  // elements per workgroup

struct AdamTable {
  float* p[ADAM_MAX_TENSORS];
  const float* g[ADAM_MAX_TENSORS];
  float* m[ADAM_MAX_TENSORS];
  float* v[ADAM_MAX_TENSORS];
  long long n[ADAM_MAX_TENSORS];
  float neg_step_size[ADAM_MAX_TENSORS];  // -(lr / (1 - b1^t)), per tensor (per-group lr and step)
  float bc2_sqrt[ADAM_MAX_TENSORS];       // sqrt(1 - b2^t)
  int first_chunk[ADAM_MAX_TENSORS + 1];  // prefix sum of chunk counts
  int count;
};

__device__ __forceinline__ void adam_update(float& p, float g, float& m, float& v, float b1, float omb1, float b2,
                                            float omb2, float eps, float neg_step, float bc2s) {
  m = m * b1 + omb1 * g;
  v = v * b2 + (omb2 * g) * g;
  const float denom = sqrtf(v) / bc2s + eps;
  p = p + (neg_step * m) / denom;
}

__global__ void __launch_bounds__(ADAM_THREADS)
adam_kernel(const AdamTable t, float b1, float omb1, float b2, float omb2, float eps, float grad_scale) {
  // which tensor does this workgroup belong to (the table is tiny and uniform: scalar loads)
  int k = 0;
  while (k + 1 < t.count && (int)blockIdx.x >= t.first_chunk[k + 1]) k++;
  const long long n = t.n[k];
  const long long base = (long long)((int)blockIdx.x - t.first_chunk[k]) * ADAM_CHUNK;
  float* __restrict__ p = t.p[k];
  const float* __restrict__ g = t.g[k];
  float* __restrict__ m = t.m[k];
  float* __restrict__ v = t.v[k];
  const float neg_step = t.neg_step_size[k], bc2s = t.bc2_sqrt[k];
  const bool aligned = ((((uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v) & 15) == 0);
  if (aligned && base + ADAM_CHUNK <= n) {
    float4 P[ADAM_ITEMS], G[ADAM_ITEMS], M[ADAM_ITEMS], Vv[ADAM_ITEMS];
#pragma unroll
    for (int i = 0; i < ADAM_ITEMS; i++) {
      const long long e = base + ((long long)i * ADAM_THREADS + threadIdx.x) * ADAM_VEC;
      P[i] = *reinterpret_cast<const float4*>(p + e);
      G[i] = *reinterpret_cast<const float4*>(g + e);
      M[i] = *reinterpret_cast<const float4*>(m + e);
      Vv[i] = *reinterpret_cast<const float4*>(v + e);
    }
#pragma unroll
    for (int i = 0; i < ADAM_ITEMS; i++) {
      const long long e = base + ((long long)i * ADAM_THREADS + threadIdx.x) * ADAM_VEC;
      adam_update(P[i].x, G[i].x * grad_scale, M[i].x, Vv[i].x, b1, omb1, b2, omb2, eps, neg_step, bc2s);
      adam_update(P[i].y, G[i].y * grad_scale, M[i].y, Vv[i].y, b1, omb1, b2, omb2, eps, neg_step, bc2s);
      adam_update(P[i].z, G[i].z * grad_scale, M[i].z, Vv[i].z, b1, omb1, b2, omb2, eps, neg_step, bc2s);
      adam_update(P[i].w, G[i].w * grad_scale, M[i].w, Vv[i].w, b1, omb1, b2, omb2, eps, neg_step, bc2s);
      *reinterpret_cast<float4*>(p + e) = P[i];
      *reinterpret_cast<float4*>(m + e) = M[i];
      *reinterpret_cast<float4*>(v + e) = Vv[i];
    }
  } else {
    for (int i = 0; i < ADAM_ITEMS * ADAM_VEC; i++) {
      const long long e = base + (long long)i * ADAM_THREADS + threadIdx.x;
      if (e < n) {
        float pe = p[e], me = m[e], ve = v[e];
        adam_update(pe, g[e] * grad_scale, me, ve, b1, omb1, b2, omb2, eps, neg_step, bc2s);
        p[e] = pe;
        m[e] = me;
        v[e] = ve;
      }
    }
  }
}

}  // namespace

int launch_adam(int count, float* const* params, const float* const* grads, float* const* exp_avg,
                float* const* exp_avg_sq, const long long* sizes, const double* lrs, const int* steps, double beta1,
                double beta2, double eps, float grad_scale, hipStream_t stream) {
  int done = 0;
  while (done < count) {
    AdamTable t;
    int k = 0, chunks = 0;
    for (; done < count && k < ADAM_MAX_TENSORS; done++) {
      if (sizes[done] <= 0) continue;
      t.p[k] = params[done];
      t.g[k] = grads[done];
      t.m[k] = exp_avg[done];
      t.v[k] = exp_avg_sq[done];
      t.n[k] = sizes[done];
      // bias corrections in double, like the Python floats of the reference optimizer
      const double bc1 = 1.0 - pow(beta1, (double)steps[done]);
      const double bc2 = 1.0 - pow(beta2, (double)steps[done]);
      t.neg_step_size[k] = (float)(-(lrs[done] / bc1));
      t.bc2_sqrt[k] = (float)sqrt(bc2);
      t.first_chunk[k] = chunks;
      chunks += (int)((sizes[done] + ADAM_CHUNK - 1) / ADAM_CHUNK);
      k++;
    }
    if (k == 0) break;
    t.first_chunk[k] = chunks;
    t.count = k;
    hipLaunchKernelGGL(adam_kernel, dim3(chunks), dim3(ADAM_THREADS), 0, stream, t, (float)beta1,
                       (float)(1.0 - beta1), (float)beta2, (float)(1.0 - beta2), (float)eps, grad_scale);
  }
  return 0;
}

}  // namespace gs
