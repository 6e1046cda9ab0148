// Sequence mixers over ragged batches for MI355X (gfx950): multi-head
// attention over paged K/V rows with a sliding window that keeps the first
// tokens, and linear recurrences with a matrix state per head (plain and
// delta-rule form) with their prologues and epilogue.
//
// Plain C ABI (raw device pointers + a hipStream_t) so the library builds in
// seconds with hipcc alone and is loaded through ctypes. dtype codes:
// 0 = float, 1 = bfloat16. Norm statistics, rotations, scores, softmax, the
// weighted sums, decays, gates and the recurrent state are float whatever
// the storage type.

#include "serving_common.h"

namespace {

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// ------------------------------------------------------ attention prologue
// proj row = [ q (H x dim) | k (G x dim) | v (G x vdim) ] (q alone without
// own_kv). RMS norm over the WHOLE q projection and over the whole k
// projection, rotation of adjacent pairs in the first rot_dims coordinates of
// each head, rows [k ; v] into the pool.
template <typename T>
__global__ __launch_bounds__(NT) void attn_prep_k(
    const T* __restrict__ proj, int ld_proj, const float* __restrict__ wq,
    const float* __restrict__ wk, const int* __restrict__ tok_pos,
    const int* __restrict__ tok_row, const float* __restrict__ cosT,
    const float* __restrict__ sinT, T* __restrict__ pool, T* __restrict__ q_out, int H, int G,
    int dim, int vdim, int rot_dims, int own_kv, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const T* p = proj + (int64_t)t * ld_proj;
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  const int half = rot_dims >> 1;
  const float* cs = cosT + (int64_t)tok_pos[t] * half;
  const float* sn = sinT + (int64_t)tok_pos[t] * half;
  float ss = 0.f;
  for (int i = threadIdx.x; i < nq; i += NT) {
    const float v = ld(p + i);
    ss += v * v;
  }
  const float rq = rsqrtf(block_sum(ss, red) / (float)nq + eps);
  for (int i = threadIdx.x; i < nq; i += NT) {
    const int c = i % dim;
    float v = ld(p + i) * rq * wq[i];
    if (c < rot_dims) {
      const int j = i - c + (c ^ 1);
      const float o = ld(p + j) * rq * wq[j];
      const float co = cs[c >> 1], si = sn[c >> 1];
      v = (c & 1) ? v * co + o * si : v * co - o * si;
    }
    st(q_out + (int64_t)t * nq + i, v);
  }
  if (!own_kv) return;
  T* row = pool + (int64_t)tok_row[t] * (nk + nv);
  const T* pk = p + nq;
  ss = 0.f;
  for (int i = threadIdx.x; i < nk; i += NT) {
    const float v = ld(pk + i);
    ss += v * v;
  }
  const float rk = rsqrtf(block_sum(ss, red) / (float)nk + eps);
  for (int i = threadIdx.x; i < nk; i += NT) {
    const int c = i % dim;
    float v = ld(pk + i) * rk * wk[i];
    if (c < rot_dims) {
      const int j = i - c + (c ^ 1);
      const float o = ld(pk + j) * rk * wk[j];
      const float co = cs[c >> 1], si = sn[c >> 1];
      v = (c & 1) ? v * co + o * si : v * co - o * si;
    }
    st(row + i, v);
  }
  for (int i = threadIdx.x; i < nv; i += NT) row[nk + i] = pk[nk + i];
}

// ------------------------------------------------------ windowed attention
// Exact kernel: one block per (token, key/value head, key split); the query
// heads of that key/value head go in groups of WHG. The keys a token sees are
// [0, n_keep) and [lo, pos]: lo = max(0, pos - window + 1) (0 without a
// window), n_keep = min(keep_first, lo). They are walked as one virtual range
// in chunks of KC, staged through LDS; scores, online softmax and the
// weighted sum are float. With nsplit > 1 the block writes (max, sum,
// unnormalised sum) and window_attn_merge_k finishes.
constexpr int WHG = 8;
constexpr int WVPT = 2;  // value columns per thread: vdim <= WVPT * NT

template <typename T>
__global__ __launch_bounds__(NT) void window_attn_k(
    const T* __restrict__ q,     // [Ttok, H, dim]
    const T* __restrict__ pool,  // rows of G*dim keys then G*vdim values
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int maxb, int bs,
    T* __restrict__ out,       // [Ttok, H, vdim]
    float* __restrict__ part,  // [Ttok, nsplit, H, vdim + 2] when nsplit > 1
    int H, int G, int dim, int vdim, int KC, int nsplit, float scale, int window,
    int keep_first) {
  extern __shared__ float smem[];
  const int DS = dim | 1;
  float* qs = smem;              // [WHG][dim]
  float* sc = qs + WHG * dim;    // [WHG][KC]
  float* alpha = sc + WHG * KC;  // [WHG]
  float* mrun = alpha + WHG;
  float* lrun = mrun + WHG;
  T* ks = reinterpret_cast<T*>(lrun + WHG);  // [KC][DS]
  T* vs = ks + KC * DS;                      // [KC][vdim]
  const int t = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int rep = H / G;
  const int row_w = G * (dim + vdim);
  const int pos = tok_pos[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_keep = min(keep_first, lo);
  const int nkeys = n_keep + pos - lo + 1;
  const int* tab = table + (int64_t)tok_seq[t] * maxb;
  const int nchunk = (nkeys + KC - 1) / KC;
  const int cps = (nchunk + nsplit - 1) / nsplit;
  const int c_lo = split * cps, c_hi = min(nchunk, c_lo + cps);

  for (int h0 = 0; h0 < rep; h0 += WHG) {
    const int nh = min(WHG, rep - h0);
    const int hbase = g * rep + h0;
    __syncthreads();
    for (int i = tid; i < nh * dim; i += NT)
      qs[i] = ld(q + ((int64_t)t * H + hbase) * dim + i);
    if (tid < WHG) {
      mrun[tid] = -INFINITY;
      lrun[tid] = 0.f;
    }
    float acc[WHG][WVPT];
#pragma unroll
    for (int h = 0; h < WHG; ++h)
#pragma unroll
      for (int i = 0; i < WVPT; ++i) acc[h][i] = 0.f;
    for (int ch = c_lo; ch < c_hi; ++ch) {
      const int k0 = ch * KC;
      const int nk = min(KC, nkeys - k0);
      __syncthreads();
      for (int i = tid; i < nk * dim; i += NT) {
        const int kk = i / dim, c = i - kk * dim;
        const int u = k0 + kk;
        const int p = u < n_keep ? u : lo + (u - n_keep);
        const int64_t r = (int64_t)tab[p / bs] * bs + p % bs;
        ks[kk * DS + c] = pool[r * row_w + g * dim + c];
      }
      for (int i = tid; i < nk * vdim; i += NT) {
        const int kk = i / vdim, c = i - kk * vdim;
        const int u = k0 + kk;
        const int p = u < n_keep ? u : lo + (u - n_keep);
        const int64_t r = (int64_t)tab[p / bs] * bs + p % bs;
        vs[kk * vdim + c] = pool[r * row_w + G * dim + g * vdim + c];
      }
      __syncthreads();
      for (int i = tid; i < nh * KC; i += NT) {
        const int h = i / KC, kk = i - h * KC;
        float d = -INFINITY;
        if (kk < nk) {
          d = 0.f;
          const float* qh = qs + h * dim;
          const T* kr = ks + kk * DS;
          for (int c = 0; c < dim; ++c) d += qh[c] * ld(kr + c);
          d *= scale;
        }
        sc[i] = d;
      }
      __syncthreads();
      for (int h = wid; h < nh; h += NT / 64) {
        float mx = -INFINITY;
        for (int kk = lane; kk < nk; kk += 64) mx = fmaxf(mx, sc[h * KC + kk]);
        mx = wave_max(mx);
        const float m_old = mrun[h];
        const float m_new = fmaxf(m_old, mx);
        float psum = 0.f;
        for (int kk = lane; kk < nk; kk += 64) {
          const float pw = expf(sc[h * KC + kk] - m_new);
          sc[h * KC + kk] = pw;
          psum += pw;
        }
        psum = wave_sum(psum);
        if (lane == 0) {
          const float a = expf(m_old - m_new);  // 0 on the first chunk
          alpha[h] = a;
          mrun[h] = m_new;
          lrun[h] = lrun[h] * a + psum;
        }
      }
      __syncthreads();
#pragma unroll
      for (int h = 0; h < WHG; ++h) {
        if (h < nh) {
          const float a = alpha[h];
#pragma unroll
          for (int i = 0; i < WVPT; ++i) acc[h][i] *= a;
        }
      }
      for (int kk = 0; kk < nk; ++kk) {
        float c[WVPT];
#pragma unroll
        for (int i = 0; i < WVPT; ++i) {
          const int col = tid + i * NT;
          c[i] = col < vdim ? ld(vs + kk * vdim + col) : 0.f;
        }
#pragma unroll
        for (int h = 0; h < WHG; ++h) {
          if (h < nh) {
            const float pw = sc[h * KC + kk];
#pragma unroll
            for (int i = 0; i < WVPT; ++i) acc[h][i] += pw * c[i];
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < WHG; ++h) {
      if (h < nh) {
        if (nsplit == 1) {
          const float inv = 1.f / lrun[h];
#pragma unroll
          for (int i = 0; i < WVPT; ++i) {
            const int col = tid + i * NT;
            if (col < vdim) st(out + ((int64_t)t * H + hbase + h) * vdim + col, acc[h][i] * inv);
          }
        } else {
          float* pp = part + (((int64_t)t * nsplit + split) * H + hbase + h) * (vdim + 2);
          if (tid == 0) {
            pp[0] = mrun[h];
            pp[1] = lrun[h];
          }
#pragma unroll
          for (int i = 0; i < WVPT; ++i) {
            const int col = tid + i * NT;
            if (col < vdim) pp[2 + col] = acc[h][i];
          }
        }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void window_attn_merge_k(
    const float* __restrict__ part, T* __restrict__ out, int H, int vdim, int nsplit) {
  const int t = blockIdx.x, h = blockIdx.y;
  float m = -INFINITY;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
    if (pp[1] > 0.f) m = fmaxf(m, pp[0]);
  }
  float l = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
    if (pp[1] > 0.f) l += pp[1] * expf(pp[0] - m);
  }
  for (int c = threadIdx.x; c < vdim; c += NT) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float* pp = part + (((int64_t)t * nsplit + s) * H + h) * (vdim + 2);
      if (pp[1] > 0.f) a += pp[2 + c] * expf(pp[0] - m);
    }
    st(out + ((int64_t)t * H + h) * vdim + c, a / l);
  }
}

// -------------------------------------------------- delta-rule prologue
// proj row = [ q (G x dim) | k (G x dim) | v (H x vdim) | gate | b (H) | a (H) ].
// One block per token: causal convolution + SiLU over the q|k|v channels
// (earlier inputs from this step's rows, from the slot's tail, or zero before
// position 0), q and k to unit length per head (q also times dim^-1/2),
// beta = sigmoid(b), decay = exp(-exp(A_log) * softplus(a + dt_bias)).
constexpr int MAXTAPS_SEQ = 32;

template <typename T>
__global__ __launch_bounds__(NT) void delta_prep_k(
    const T* __restrict__ proj, int ld_proj, const T* __restrict__ w,
    const T* __restrict__ state, int64_t state_slot_stride, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ q_out, float* __restrict__ k_out,
    float* __restrict__ v_out, float* __restrict__ beta, float* __restrict__ decay, int G, int H,
    int dim, int vdim, int taps) {
  extern __shared__ float ys[];  // [2*G*dim] conv outputs of q and k
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int j = t - cu[s];
  const int pos = tok_pos[t];
  const int tail = taps - 1;
  const int nqk = G * dim, nv = H * vdim;
  const int C = 2 * nqk + nv;
  const T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  const T* p = proj + (int64_t)t * ld_proj;
  for (int c = threadIdx.x; c < C; c += NT) {
    float acc = ld(w + (int64_t)c * taps + tail) * ld(p + c);
    for (int k = 1; k < taps; ++k) {
      if (pos - k < 0) break;
      const float hk = k <= j ? ld(p - (int64_t)k * ld_proj + c)
                              : ld(sl + (int64_t)(tail + j - k) * C + c);
      acc += ld(w + (int64_t)c * taps + tail - k) * hk;
    }
    const float y = siluf_(acc);
    if (c < 2 * nqk)
      ys[c] = y;
    else
      v_out[(int64_t)t * nv + c - 2 * nqk] = y;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const float qscale = rsqrtf((float)dim);
  for (int hd = wid; hd < 2 * G; hd += NT / 64) {
    const float* y = ys + hd * dim;
    float ss = 0.f;
    for (int c = lane; c < dim; c += 64) ss += y[c] * y[c];
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss + 1e-6f) * (hd < G ? qscale : 1.f);
    float* o = hd < G ? q_out + ((int64_t)t * G + hd) * dim
                      : k_out + ((int64_t)t * G + hd - G) * dim;
    for (int c = lane; c < dim; c += 64) o[c] = y[c] * inv;
  }
  for (int h = threadIdx.x; h < H; h += NT) {
    beta[(int64_t)t * H + h] = sigmoidf_(ld(p + C + nv + h));
    const float dt = softplusf_(ld(p + C + nv + H + h) + dt_bias[h]);
    decay[(int64_t)t * H + h] = expf(-expf(a_log[h]) * dt);
  }
}

// One block per sequence: the tail becomes the sequence's last taps-1 inputs
// (from this step's rows, or shifted out of the old tail for short steps).
template <typename T>
__global__ __launch_bounds__(NT) void conv_tail_shift_k(
    const T* __restrict__ x, int ld_x, T* __restrict__ state, int64_t state_slot_stride,
    const int* __restrict__ cu, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, int C, int taps) {
  const int s = blockIdx.x;
  const int tail = taps - 1;
  const int start = seq_start[s];
  const int count = cu[s + 1] - cu[s];
  T* sl = state + (int64_t)seq_slot[s] * state_slot_stride;
  for (int c = threadIdx.x; c < C; c += NT) {
    for (int i = 0; i < tail; ++i) {  // ascending: reads stay ahead of writes
      const int p = start + count - tail + i;  // position kept at i
      T v;
      if (p >= start)
        v = x[(int64_t)(cu[s] + p - start) * ld_x + c];
      else if (p >= 0)
        v = sl[(int64_t)(i + count) * C + c];
      else
        st(&v, 0.f);
      sl[(int64_t)i * C + c] = v;
    }
  }
}

// sigmoid(z + bias)^inv_tau = exp(inv_tau * log_sigmoid(z + bias))
template <typename T>
__global__ void sigmoid_pow_k(const T* __restrict__ z, const float* __restrict__ bias,
                              float* __restrict__ out, int64_t n, int C, float inv_tau) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float x = ld(z + i) + bias[i % C];
    const float ls = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
    out[i] = expf(inv_tau * ls);
  }
}

// ------------------------------------------------------ linear recurrence
// S [dim, vdim] per (slot, head), float. The columns of S are independent in
// both forms, so the work is split by column: SCAN_R lanes share a column,
// each holding ROWS consecutive rows of it in registers (dim <= SCAN_R * ROWS,
// rows beyond dim stay zero); a block of NT threads owns NT / SCAN_R columns of
// one head of one sequence and walks the sequence's tokens in order:
//   S *= decay; d = S^T k; u = DELTA ? beta * (v - d) : v; S += k u; o = S^T q.
// Sums over rows go lane-local first, then across the SCAN_R lanes in a fixed
// order, so a result does not depend on where a sequence was cut. The next
// token's operands are loaded while the current one is computed.
constexpr int SCAN_R = 8;
constexpr int SCAN_COLS = NT / SCAN_R;

__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
  for (int o = 1; o < SCAN_R; o <<= 1) x += __shfl_xor(x, o, 64);
  return x;
}

template <typename T, int ROWS, bool DELTA, bool CHANNEL_DECAY>
__global__ __launch_bounds__(NT) void linear_scan_k(
    const T* __restrict__ q, int ld_q, const T* __restrict__ k, int ld_k,
    const T* __restrict__ v, int ld_v, const float* __restrict__ decay,
    const float* __restrict__ beta, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ seq_slot, float* __restrict__ out, int G, int H, int dim, int vdim,
    float q_scale) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int r = threadIdx.x % SCAN_R;
  const int col = blockIdx.z * SCAN_COLS + threadIdx.x / SCAN_R;
  const bool live = col < vdim;
  const int cc = live ? col : vdim - 1;  // idle lanes shadow the last column
  const int g = h / (H / G);
  const int r0 = r * ROWS;
  float* Sg = state + (((int64_t)seq_slot[s] * H + h) * dim) * vdim + cc;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = r0 + i < dim ? Sg[(int64_t)(r0 + i) * vdim] : 0.f;
  const int t0 = cu[s], t1 = cu[s + 1];
  float kn[ROWS], qn[ROWS], dn[CHANNEL_DECAY ? ROWS : 1], vn = 0.f, bn = 1.f;
  auto fetch = [&](int t) {
    const T* kp = k + (int64_t)t * ld_k + g * dim + r0;
    const T* qp = q + (int64_t)t * ld_q + g * dim + r0;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const bool in = r0 + i < dim;
      kn[i] = in ? ld(kp + i) : 0.f;
      qn[i] = in ? ld(qp + i) * q_scale : 0.f;
    }
    if (CHANNEL_DECAY) {
      const float* dp = decay + ((int64_t)t * H + h) * dim + r0;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) dn[i] = r0 + i < dim ? dp[i] : 0.f;
    } else {
      dn[0] = decay[(int64_t)t * H + h];
    }
    vn = ld(v + (int64_t)t * ld_v + h * vdim + cc);
    if (DELTA) bn = beta[(int64_t)t * H + h];
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float kc[ROWS], qc[ROWS], dc[CHANNEL_DECAY ? ROWS : 1];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      kc[i] = kn[i];
      qc[i] = qn[i];
    }
#pragma unroll
    for (int i = 0; i < (CHANNEL_DECAY ? ROWS : 1); ++i) dc[i] = dn[i];
    const float vc = vn, bc = bn;
    if (t + 1 < t1) fetch(t + 1);
    float u = vc;
    if (DELTA) {
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        S[i] *= CHANNEL_DECAY ? dc[i] : dc[0];
        d += S[i] * kc[i];
      }
      u = bc * (vc - group_sum(d));
    } else {
#pragma unroll
      for (int i = 0; i < ROWS; ++i) S[i] *= CHANNEL_DECAY ? dc[i] : dc[0];
    }
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      S[i] += kc[i] * u;
      o += S[i] * qc[i];
    }
    o = group_sum(o);
    if (live && r == 0) out[((int64_t)t * H + h) * vdim + col] = o;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (r0 + i < dim) Sg[(int64_t)(r0 + i) * vdim] = S[i];
  }
}

// out[t, h*vdim + c] = o / sqrt(mean_c(o^2) + eps) * w[c] * silu(gate)
template <typename T>
__global__ __launch_bounds__(NT) void head_norm_gate_k(
    const float* __restrict__ o, const float* __restrict__ w, const T* __restrict__ gate,
    int ld_gate, T* __restrict__ out, int H, int vdim, float eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  for (int h = wid; h < H; h += NT / 64) {
    const float* oh = o + ((int64_t)t * H + h) * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) ss += oh[c] * oh[c];
    const float inv = rsqrtf(wave_sum(ss) / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64) {
      const float gv = ld(gate + (int64_t)t * ld_gate + h * vdim + c);
      st(out + ((int64_t)t * H + h) * vdim + c, oh[c] * inv * w[c] * siluf_(gv));
    }
  }
}

}  // namespace

extern "C" {

int dsv_attn_prep(const void* proj, int ld_proj, const float* wq, const float* wk,
                  const int* tok_pos, const int* tok_row, const float* cosT, const float* sinT,
                  void* pool, void* q_out, int dt, int Ttok, int H, int G, int dim, int vdim,
                  int rot_dims, int own_kv, float eps, hipStream_t s) {
  if (rot_dims < 0 || (rot_dims & 1) || rot_dims > dim || H % G) return -1;
  if (Ttok <= 0) return 0;
  BY_DTYPE(dt, (attn_prep_k<T><<<Ttok, NT, 0, s>>>((const T*)proj, ld_proj, wq, wk, tok_pos,
                                                   tok_row, cosT, sinT, (T*)pool, (T*)q_out, H,
                                                   G, dim, vdim, rot_dims, own_kv, eps)));
  return (int)hipGetLastError();
}

// LDS bytes of the exact attention kernel for a chunk of KC keys
int64_t dsv_window_attn_lds(int dt, int dim, int vdim, int KC) {
  return (int64_t)(WHG * dim + WHG * KC + 3 * WHG) * 4 +
         (int64_t)KC * ((dim | 1) + vdim) * (dt == 0 ? 4 : 2);
}

int dsv_window_attn(const void* q, const void* pool, const int* tok_seq, const int* tok_pos,
                    const int* table, int maxb, int bs, void* out, float* part, int dt, int Ttok,
                    int H, int G, int dim, int vdim, int KC, int nsplit, float scale, int window,
                    int keep_first, hipStream_t s) {
  if (vdim > WVPT * NT || H % G || nsplit < 1 || (nsplit > 1 && !part)) return -1;
  if (Ttok <= 0) return 0;
  const int64_t lds = dsv_window_attn_lds(dt, dim, vdim, KC);
  if (lds > 64 * 1024) return -2;
  dim3 grid(Ttok, G, nsplit);
  BY_DTYPE(dt, (window_attn_k<T><<<grid, NT, lds, s>>>(
                   (const T*)q, (const T*)pool, tok_seq, tok_pos, table, maxb, bs, (T*)out, part,
                   H, G, dim, vdim, KC, nsplit, scale, window, keep_first)));
  if (nsplit > 1) {
    dim3 g2(Ttok, H);
    BY_DTYPE(dt, (window_attn_merge_k<T><<<g2, NT, 0, s>>>(part, (T*)out, H, vdim, nsplit)));
  }
  return (int)hipGetLastError();
}

int dsv_delta_prep(const void* proj, int ld_proj, const void* w, void* state,
                   int64_t state_slot_stride, const int* cu, const int* seq_slot,
                   const int* seq_start, const int* tok_seq, const int* tok_pos,
                   const float* a_log, const float* dt_bias, float* q_out, float* k_out,
                   float* v_out, float* beta, float* decay, int dt, int Ttok, int nseq, int G,
                   int H, int dim, int vdim, int taps, hipStream_t s) {
  if (taps < 1 || taps > MAXTAPS_SEQ || H % G) return -1;
  if (Ttok <= 0) return 0;
  const int64_t lds = (int64_t)2 * G * dim * 4;
  if (lds > 64 * 1024) return -2;
  const int C = 2 * G * dim + H * vdim;
  BY_DTYPE(dt, (delta_prep_k<T><<<Ttok, NT, lds, s>>>(
                   (const T*)proj, ld_proj, (const T*)w, (const T*)state, state_slot_stride, cu,
                   seq_slot, tok_seq, tok_pos, a_log, dt_bias, q_out, k_out, v_out, beta, decay,
                   G, H, dim, vdim, taps)));
  if (taps > 1)
    BY_DTYPE(dt, (conv_tail_shift_k<T><<<nseq, NT, 0, s>>>((const T*)proj, ld_proj, (T*)state,
                                                           state_slot_stride, cu, seq_slot,
                                                           seq_start, C, taps)));
  return (int)hipGetLastError();
}

int dsv_sigmoid_pow(const void* z, const float* bias, float* out, int dt, int64_t n, int C,
                    float inv_tau, hipStream_t s) {
  if (n <= 0) return 0;
  BY_DTYPE(dt, (sigmoid_pow_k<T><<<nblocks(n, 256), 256, 0, s>>>((const T*)z, bias, out, n, C,
                                                                 inv_tau)));
  return (int)hipGetLastError();
}

// largest head size of keys the scan covers
int dsv_linear_scan_max_dim() { return SCAN_R * 32; }

// q/k/v: dtype dt with row strides in elements; decay [T, H] (channel_decay 0)
// or [T, H, dim]; beta [T, H] or null (plain form).
int dsv_linear_scan(const void* q, int ld_q, const void* k, int ld_k, const void* v, int ld_v,
                    const float* decay, int channel_decay, const float* beta, float* state,
                    const int* cu, const int* seq_slot, float* out, int dt, int nseq, int G, int H,
                    int dim, int vdim, float q_scale, hipStream_t s) {
  if (dim > dsv_linear_scan_max_dim() || dim < 1 || H % G) return -1;
  if (nseq <= 0) return 0;
  dim3 grid(nseq, H, (vdim + SCAN_COLS - 1) / SCAN_COLS);
#define SCAN(ROWS, DELTA, CD)                                                                   \
  BY_DTYPE(dt, (linear_scan_k<T, ROWS, DELTA, CD><<<grid, NT, 0, s>>>(                           \
                   (const T*)q, ld_q, (const T*)k, ld_k, (const T*)v, ld_v, decay, beta, state,  \
                   cu, seq_slot, out, G, H, dim, vdim, q_scale)))
#define SCAN_BY_ROWS(DELTA, CD)                   \
  do {                                            \
    if (dim <= SCAN_R * 4) SCAN(4, DELTA, CD);    \
    else if (dim <= SCAN_R * 8) SCAN(8, DELTA, CD);   \
    else if (dim <= SCAN_R * 16) SCAN(16, DELTA, CD); \
    else SCAN(32, DELTA, CD);                     \
  } while (0)
  if (beta && channel_decay) SCAN_BY_ROWS(true, true);
  else if (beta) SCAN_BY_ROWS(true, false);
  else if (channel_decay) SCAN_BY_ROWS(false, true);
  else SCAN_BY_ROWS(false, false);
#undef SCAN_BY_ROWS
#undef SCAN
  return (int)hipGetLastError();
}

int dsv_head_norm_gate(const float* o, const float* w, const void* gate, int ld_gate, void* out,
                       int dt, int Ttok, int H, int vdim, float eps, hipStream_t s) {
  if (Ttok <= 0) return 0;
  BY_DTYPE(dt, (head_norm_gate_k<T><<<Ttok, NT, 0, s>>>(o, w, (const T*)gate, ld_gate, (T*)out, H,
                                                        vdim, eps)));
  return (int)hipGetLastError();
}

}  // extern "C"
