// The gated delta rule: a linear-attention mixer with one fp32 state matrix per head and request.
//
//   per head and token:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// q, k [dk] and v [dv] come from projections that pass a short causal convolution over time (one
// filter per channel, `taps` taps, the last tap on the current token) and silu; q and k are made unit
// vectors per head (q also times dk^-1/2); beta = sigmoid(b); g = exp(-exp(A_log) softplus(a + dt_bias)).
// A request's state row holds S of every head ([H, dk, dv]) and behind it the last taps - 1 inputs of
// the convolution ([taps - 1, C], oldest first), all fp32.  Everything here is fp32 arithmetic; only the
// projections' storage type is templated.
//
// Four kernels a step: (1) convolution + silu + unit vectors + beta and g for every token, in
// parallel; (2) the convolution's new state; (3) the recurrence, a workgroup per (segment, head, tile
// of columns of S), token after token; (4) the read-out's norm per head times the output gate.
#include "common.h"

#define DR_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ---------------------------------------------------------------------------------------------
// (1) z [T, zs]: columns [q: Hk dk | k: Hk dk | v: H dv | ...]; the first C = 2 Hk dk + H dv of
// them are the convolution's channels.  grid (T, 2 Hk + H + 1): a workgroup of 64 threads per token
// and head of q, k or v, and one for the token's beta and g.
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(64) void delta_prepare_kernel(
    const TA* __restrict__ z, int zs, const float* __restrict__ conv_w, const float* __restrict__ state,
    size_t state_stride, size_t conv_off, const float* __restrict__ ba, const float* __restrict__ A_log,
    const float* __restrict__ dt_bias, const int* __restrict__ seg_of_token, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vc,
    float* __restrict__ beta, float* __restrict__ decay, int H, int Hk, int dk, int dv, int taps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int u = blockIdx.y;
  if (u == 2 * Hk + H) {
    for (int h = threadIdx.x; h < H; h += blockDim.x) {
      const float b = ba[(size_t)t * 2 * H + h];
      const float a = ba[(size_t)t * 2 * H + H + h];
      beta[(size_t)t * H + h] = 1.f / (1.f + expf(-b));
      decay[(size_t)t * H + h] = expf(-expf(A_log[h]) * softplus_f(a + dt_bias[h]));
    }
    return;
  }
  const int seg = seg_of_token[t];
  const int t0 = cu_q[seg];
  const int slot = state_slots[seg];
  const int C = 2 * Hk * dk + H * dv;
  int c0, n, kind;
  float* dst;
  if (u < Hk) { kind = 0; n = dk; c0 = u * dk; dst = qn + ((size_t)t * Hk + u) * dk; }
  else if (u < 2 * Hk) { kind = 1; n = dk; c0 = Hk * dk + (u - Hk) * dk; dst = kn + ((size_t)t * Hk + (u - Hk)) * dk; }
  else { kind = 2; n = dv; c0 = 2 * Hk * dk + (u - 2 * Hk) * dv; dst = vc + ((size_t)t * H + (u - 2 * Hk)) * dv; }
  const float* cs = slot >= 0 ? state + (size_t)slot * state_stride + conv_off : nullptr;
  float vals[4];          // n <= 256
  float ss = 0.f;
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int i = threadIdx.x + m * 64;
    float y = 0.f;
    if (i < n) {
      const int c = c0 + i;
      float acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int tp = t - (taps - 1 - j);
        float xv;
        if (tp >= t0) xv = to_float(z[(size_t)tp * zs + c]);
        else xv = cs ? cs[(size_t)(taps - 1 + tp - t0) * C + c] : 0.f;
        acc += conv_w[(size_t)c * taps + j] * xv;
      }
      y = silu_f(acc);
    }
    vals[m] = y;
    ss += y * y;
  }
  float scale = 1.f;
  if (kind != 2) {
    ss = block_sum(ss, scratch);
    scale = 1.f / sqrtf(ss + 1e-6f);
    if (kind == 0) scale *= 1.f / sqrtf((float)dk);
  }
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int i = threadIdx.x + m * 64;
    if (i < n) dst[i] = vals[m] * scale;
  }
}

// ---------------------------------------------------------------------------------------------
// (2) the last taps - 1 inputs of every channel after the step: from the step's own tokens, and
// from the old state where the segment brought fewer than taps - 1.  grid (B, ceil(C / 256)).
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void delta_conv_state_kernel(
    const TA* __restrict__ z, int zs, float* __restrict__ state, size_t state_stride, size_t conv_off,
    const int* __restrict__ cu_q, const int* __restrict__ state_slots, int C, int taps) {
  const int seg = blockIdx.x;
  const int slot = state_slots[seg];
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (slot < 0 || c >= C) return;
  const int t0 = cu_q[seg], n = cu_q[seg + 1] - t0;
  float* cs = state + (size_t)slot * state_stride + conv_off;
  float nv[DR_MAX_TAPS - 1];
#pragma unroll
  for (int i = 0; i < DR_MAX_TAPS - 1; ++i) {
    if (i < taps - 1) {
      const int li = n - (taps - 1) + i;
      nv[i] = li >= 0 ? to_float(z[(size_t)(t0 + li) * zs + c]) : cs[(size_t)(i + n) * C + c];
    }
  }
#pragma unroll
  for (int i = 0; i < DR_MAX_TAPS - 1; ++i)
    if (i < taps - 1) cs[(size_t)i * C + c] = nv[i];
}

// ---------------------------------------------------------------------------------------------
// (3) the recurrence.  grid (ceil(dv / cols), H, B).  A column of S is cut in R parts along dk: a thread
// keeps RPT rows of one column in registers, so that S^T k and S^T q are sums inside a thread plus
// log2(R) exchanges between neighbouring lanes.  R = 4 (a wave holds 16 columns) for steps of single
// tokens, where reading and writing the state is the work and neighbouring lanes should touch
// neighbouring columns; R = 16 (a wave holds 4 columns, a head is spread over four times as many waves)
// for prompt portions, where the tokens of a segment form one chain of dependent steps and the length of
// a step is what counts.  The tokens of a segment come through LDS in chunks of CH; a segment's state is
// read once and written once.
// ---------------------------------------------------------------------------------------------
// The sum of v over groups of R neighbouring lanes (R = 4 or 16), in every lane of the group, by data-parallel
// moves inside a row of 16 lanes: neighbours, pairs of neighbours, then the mirrored half and the mirrored row
// (every lane of a group of four, then of eight, already holds its group's sum, so mirrors serve as well as swaps).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int R>
__device__ __forceinline__ float lanes_sum(float v) {
  static_assert(R == 4 || R == 16, "groups of 4 or 16 lanes");
  v += dpp_move<0xB1>(v);          // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);          // quad_perm [2, 3, 0, 1]
  if (R == 16) {
    v += dpp_move<0x141>(v);       // row_half_mirror
    v += dpp_move<0x140>(v);       // row_mirror
  }
  return v;
}

template <int RPT, int R, int CH>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vc,
    const float* __restrict__ beta, const float* __restrict__ decay, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
    float* __restrict__ o, int H, int Hk, int dk, int dv) {
  constexpr int PAD = RPT + 4;           // a part's rows in LDS, padded so that neighbouring parts lie in other banks
  constexpr int ROW = R * PAD;
  __shared__ __attribute__((aligned(16))) float sq[CH][ROW];
  __shared__ __attribute__((aligned(16))) float sk[CH][ROW];
  __shared__ float sv[CH][256 / R];
  __shared__ float sb[CH], sg[CH];
  const int cols = blockDim.x / R;
  const int cl = threadIdx.x / R, r = threadIdx.x % R;
  const int j = blockIdx.x * cols + cl;
  const int h = blockIdx.y, seg = blockIdx.z;
  const int hk = h / (H / Hk);
  const bool active = j < dv;
  const int slot = state_slots[seg];
  const int t0 = cu_q[seg], n = cu_q[seg + 1] - t0;
  float* st = slot >= 0 ? state + (size_t)slot * state_stride + (size_t)h * dk * dv : nullptr;
  float S[RPT];
#pragma unroll
  for (int ii = 0; ii < RPT; ++ii) {
    const int i = r * RPT + ii;
    S[ii] = (st && active && i < dk) ? st[(size_t)i * dv + j] : 0.f;
  }
  for (int c0 = 0; c0 < n; c0 += CH) {
    const int m = min(CH, n - c0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < m * R * RPT; idx += blockDim.x) {
      const int tt = idx / (R * RPT), i = idx - tt * (R * RPT);
      const int pos = (i / RPT) * PAD + (i % RPT);
      const bool in = i < dk;
      const size_t src = ((size_t)(t0 + c0 + tt) * Hk + hk) * dk + i;
      sq[tt][pos] = in ? qn[src] : 0.f;
      sk[tt][pos] = in ? kn[src] : 0.f;
    }
    for (int idx = threadIdx.x; idx < m * cols; idx += blockDim.x) {
      const int tt = idx / cols, c = idx - tt * cols;
      const int jj = blockIdx.x * cols + c;
      sv[tt][c] = jj < dv ? vc[((size_t)(t0 + c0 + tt) * H + h) * dv + jj] : 0.f;
    }
    if (threadIdx.x < m) {
      const int tt = threadIdx.x;
      sb[tt] = beta[(size_t)(t0 + c0 + tt) * H + h];
      sg[tt] = decay[(size_t)(t0 + c0 + tt) * H + h];
    }
    __syncthreads();
    // One pass over the thread's rows a token: with Sd = g S, a = Sd^T k and c = Sd^T q are summed side by
    // side (and k.q with them), u = beta (v - a), the read-out of the updated state is c + u (k.q), and
    // S = Sd + k u.  The three sums cross the R lanes together; the next token's k and q are fetched from
    // LDS before this token's sums are awaited.
    float kreg[RPT], qreg[RPT];
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii) {
      kreg[ii] = sk[0][r * PAD + ii];
      qreg[ii] = sq[0][r * PAD + ii];
    }
    for (int tt = 0; tt < m; ++tt) {
      const float g = sg[tt], b = sb[tt], vj = sv[tt][cl];
      float a4[4] = {0.f, 0.f, 0.f, 0.f}, c4[4] = {0.f, 0.f, 0.f, 0.f}, p4[4] = {0.f, 0.f, 0.f, 0.f};
      float kcur[RPT];
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii) {
        kcur[ii] = kreg[ii];
        S[ii] *= g;
        a4[ii & 3] += S[ii] * kreg[ii];
        c4[ii & 3] += S[ii] * qreg[ii];
        p4[ii & 3] += kreg[ii] * qreg[ii];
      }
      const int nx = min(tt + 1, m - 1);
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii) {
        kreg[ii] = sk[nx][r * PAD + ii];
        qreg[ii] = sq[nx][r * PAD + ii];
      }
      const float a = lanes_sum<R>((a4[0] + a4[1]) + (a4[2] + a4[3]));
      const float c = lanes_sum<R>((c4[0] + c4[1]) + (c4[2] + c4[3]));
      const float kq = lanes_sum<R>((p4[0] + p4[1]) + (p4[2] + p4[3]));
      const float u = b * (vj - a);
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii) S[ii] += kcur[ii] * u;
      if (r == 0 && active) o[((size_t)(t0 + c0 + tt) * H + h) * dv + j] = c + u * kq;
    }
  }
  if (st && active) {
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii) {
      const int i = r * RPT + ii;
      if (i < dk) st[(size_t)i * dv + j] = S[ii];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// (3b) the recurrence for prompt portions, four tokens a pass.  With S0 the state before tokens 0..3 of a
// block, G_i = g_0 .. g_i and r_li = g_(l+1) .. g_i:
//     a_i = G_i S0^T k_i + sum_(l<i)  r_li u_l (k_l . k_i)          u_i = beta_i (v_i - a_i)
//     o_i = G_i S0^T q_i + sum_(l<=i) r_li u_l (k_l . q_i)          S  = G_3 S0 + sum_l r_l3 k_l u_l^T
// so one pass over the thread's rows gives the eight sums S0^T k_i, S0^T q_i, one exchange between the lanes
// carries all eight, the four u_i follow from scalars alone, and a second pass writes the new state: the
// chain of dependent steps is a quarter as long as token by token.  The products k_l . k_i and k_l . q_i do
// not depend on the state: they are taken once per chunk, from LDS, for all columns.  A block that the
// segment's end cuts short is filled with tokens that change nothing (k = q = 0, beta = 0, g = 1).
// ---------------------------------------------------------------------------------------------
template <int RPT, int CH>
__global__ __launch_bounds__(256) void delta_recurrence_block_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vc,
    const float* __restrict__ beta, const float* __restrict__ decay, float* __restrict__ state,
    size_t state_stride, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
    float* __restrict__ o, int H, int Hk, int dk, int dv) {
  constexpr int R = 16;
  constexpr int PAD = RPT + 4;
  constexpr int ROW = R * PAD;
  constexpr int NB = CH / 4;
  static_assert(CH % 4 == 0, "chunks are whole blocks of four");
  __shared__ __attribute__((aligned(16))) float sq[CH][ROW];
  __shared__ __attribute__((aligned(16))) float sk[CH][ROW];
  __shared__ float sv[CH][16];
  __shared__ float sb[CH], sg[CH];
  __shared__ float skk[NB][6];           // k_l . k_i, l < i:  (0,1) (0,2) (0,3) (1,2) (1,3) (2,3)
  __shared__ float skq[NB][10];          // k_l . q_i, l <= i: (0,0) (0,1) (0,2) (0,3) (1,1) (1,2) (1,3) (2,2) (2,3) (3,3)
  const int cols = blockDim.x / R;
  const int cl = threadIdx.x / R, r = threadIdx.x % R;
  const int j = blockIdx.x * cols + cl;
  const int h = blockIdx.y, seg = blockIdx.z;
  const int hk = h / (H / Hk);
  const bool active = j < dv;
  const int slot = state_slots[seg];
  const int t0 = cu_q[seg], n = cu_q[seg + 1] - t0;
  float* st = slot >= 0 ? state + (size_t)slot * state_stride + (size_t)h * dk * dv : nullptr;
  float S[RPT];
#pragma unroll
  for (int ii = 0; ii < RPT; ++ii) {
    const int i = r * RPT + ii;
    S[ii] = (st && active && i < dk) ? st[(size_t)i * dv + j] : 0.f;
  }
  for (int c0 = 0; c0 < n; c0 += CH) {
    const int m = min(CH, n - c0);
    const int mpad = (m + 3) & ~3;
    __syncthreads();
    for (int idx = threadIdx.x; idx < mpad * R * RPT; idx += blockDim.x) {
      const int tt = idx / (R * RPT), i = idx - tt * (R * RPT);
      const int pos = (i / RPT) * PAD + (i % RPT);
      const bool in = tt < m && i < dk;
      const size_t src = ((size_t)(t0 + c0 + min(tt, m - 1)) * Hk + hk) * dk + min(i, dk - 1);
      const float qv = qn[src], kv = kn[src];
      sq[tt][pos] = in ? qv : 0.f;
      sk[tt][pos] = in ? kv : 0.f;
    }
    for (int idx = threadIdx.x; idx < mpad * cols; idx += blockDim.x) {
      const int tt = idx / cols, c = idx - tt * cols;
      const int jj = blockIdx.x * cols + c;
      sv[tt][c] = (tt < m && jj < dv) ? vc[((size_t)(t0 + c0 + tt) * H + h) * dv + jj] : 0.f;
    }
    if (threadIdx.x < mpad) {
      const int tt = threadIdx.x;
      sb[tt] = tt < m ? beta[(size_t)(t0 + c0 + tt) * H + h] : 0.f;
      sg[tt] = tt < m ? decay[(size_t)(t0 + c0 + tt) * H + h] : 1.f;
    }
    __syncthreads();
    // the state-free products of every block of the chunk: sixteen a block, one per group of R lanes and pass
    // (a lane sums its part of the rows, the group adds up)
    for (int id = cl; id < (mpad / 4) * 16; id += cols) {
      const int blk = id >> 4, which = id & 15;
      const int l = (int)((0xe9500940ull >> (2 * which)) & 3), i = (int)((0xfb9e4fb9ull >> (2 * which)) & 3);
      const float* kl = &sk[blk * 4 + l][r * PAD];
      const float* xi = which >= 6 ? &sq[blk * 4 + i][r * PAD] : &sk[blk * 4 + i][r * PAD];
      float dsum = 0.f;
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii) dsum += kl[ii] * xi[ii];
      dsum = lanes_sum<R>(dsum);
      if (r == 0) {
        if (which >= 6) skq[blk][which - 6] = dsum;
        else skk[blk][which] = dsum;
      }
    }
    __syncthreads();
    for (int bb = 0; bb < mpad / 4; ++bb) {
      const int tb = bb * 4;
      float A[4] = {0.f, 0.f, 0.f, 0.f}, C[4] = {0.f, 0.f, 0.f, 0.f};
      float kr[4][RPT];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int ii = 0; ii < RPT; ++ii) {
          kr[i][ii] = sk[tb + i][r * PAD + ii];
          A[i] += S[ii] * kr[i][ii];
          C[i] += S[ii] * sq[tb + i][r * PAD + ii];
        }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        A[i] = lanes_sum<R>(A[i]);
        C[i] = lanes_sum<R>(C[i]);
      }
      const float g0 = sg[tb], g1 = sg[tb + 1], g2 = sg[tb + 2], g3 = sg[tb + 3];
      const float G0 = g0, G1 = g0 * g1, G2 = G1 * g2, G3 = G2 * g3;
      const float r01 = g1, r02 = g1 * g2, r03 = r02 * g3, r12 = g2, r13 = g2 * g3, r23 = g3;
      const float* kk = skk[bb];
      const float* kq = skq[bb];
      const float u0 = sb[tb] * (sv[tb][cl] - G0 * A[0]);
      const float u1 = sb[tb + 1] * (sv[tb + 1][cl] - (G1 * A[1] + r01 * u0 * kk[0]));
      const float u2 = sb[tb + 2] * (sv[tb + 2][cl] - (G2 * A[2] + r02 * u0 * kk[1] + r12 * u1 * kk[3]));
      const float u3 = sb[tb + 3] * (sv[tb + 3][cl] - (G3 * A[3] + r03 * u0 * kk[2] + r13 * u1 * kk[4] + r23 * u2 * kk[5]));
      const float o0 = G0 * C[0] + u0 * kq[0];
      const float o1 = G1 * C[1] + r01 * u0 * kq[1] + u1 * kq[4];
      const float o2 = G2 * C[2] + r02 * u0 * kq[2] + r12 * u1 * kq[5] + u2 * kq[7];
      const float o3 = G3 * C[3] + r03 * u0 * kq[3] + r13 * u1 * kq[6] + r23 * u2 * kq[8] + u3 * kq[9];
      const float w0 = r03 * u0, w1 = r13 * u1, w2 = r23 * u2;
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii)
        S[ii] = G3 * S[ii] + ((w0 * kr[0][ii] + w1 * kr[1][ii]) + (w2 * kr[2][ii] + u3 * kr[3][ii]));
      if (r == 0 && active) {
        float* op = o + ((size_t)(t0 + c0 + tb) * H + h) * dv + j;
        const size_t os = (size_t)H * dv;
        if (tb < m) op[0] = o0;
        if (tb + 1 < m) op[os] = o1;
        if (tb + 2 < m) op[2 * os] = o2;
        if (tb + 3 < m) op[3 * os] = o3;
      }
    }
  }
  if (st && active) {
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii) {
      const int i = r * RPT + ii;
      if (i < dk) st[(size_t)i * dv + j] = S[ii];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// (4) y[t, h, :] = o[t, h, :] / sqrt(mean(o^2) + eps) * w * silu(gate[t, h, :]); gate is a block of
// columns of z.  A wave per (token, head).
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void delta_gated_norm_kernel(const float* __restrict__ o, const TA* __restrict__ z,
                                                               int zs, int gate_col, const float* __restrict__ w,
                                                               TA* __restrict__ y, float eps, int TH, int H, int dv) {
  const int p = blockIdx.x * (blockDim.x / SA_WAVE) + threadIdx.x / SA_WAVE;
  if (p >= TH) return;
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const int t = p / H, h = p - t * H;
  const float* op = o + (size_t)p * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += SA_WAVE) ss += op[i] * op[i];
  ss = wave_sum(ss);
  const float rs = 1.f / sqrtf(ss / (float)dv + eps);
  const TA* gp = z + (size_t)t * zs + gate_col + (size_t)h * dv;
  for (int i = lane; i < dv; i += SA_WAVE)
    y[(size_t)p * dv + i] = from_float<TA>(((op[i] * rs) * w[i]) * silu_f(to_float(gp[i])));
}

// ---------------------------------------------------------------------------------------------
// One call runs the four kernels.  z: the fused projections [T, zs] = [q | k | v | gate | ...];
// ba fp32 [T, 2 H] (b then a); work: fp32 scratch of T (2 Hk dk + 2 H dv + 2 H) floats; y [T, H dv].
// ---------------------------------------------------------------------------------------------
extern "C" long long sa_delta_rule_work_floats(int T, int H, int Hk, int dk, int dv) {
  return (long long)T * (2LL * Hk * dk + 2LL * H * dv + 2LL * H);
}

extern "C" int sa_delta_rule(const void* z, int act_dtype, int zs, const float* conv_w, const float* ba,
                             const float* A_log, const float* dt_bias, const float* norm_w, float* state,
                             long long state_stride, const int* seg_of_token, const int* cu_q,
                             const int* state_slots, float* work, void* y, float eps, int T, int B, int max_q_len,
                             int H, int Hk, int dk, int dv, int taps, hipStream_t stream) {
  if (T <= 0 || B <= 0) return 0;
  if (H <= 0 || Hk <= 0 || H % Hk || dk <= 0 || dk > 256 || dv <= 0 || dv > 256 || taps < 1 || taps > DR_MAX_TAPS)
    return SA_ERR_ARG;
  if (B > 65535 || H > 65535 || 2 * Hk + H + 1 > 65535) return SA_ERR_ARG;
  const int C = 2 * Hk * dk + H * dv;
  if (zs < C + H * dv) return SA_ERR_ARG;
  const size_t conv_off = (size_t)H * dk * dv;
  if ((size_t)state_stride < conv_off + (size_t)(taps - 1) * C) return SA_ERR_ARG;
  float* qn = work;
  float* kn = qn + (size_t)T * Hk * dk;
  float* vc = kn + (size_t)T * Hk * dk;
  float* o = vc + (size_t)T * H * dv;
  float* beta = o + (size_t)T * H * dv;
  float* decay = beta + (size_t)T * H;
  {
    dim3 grid(T, 2 * Hk + H + 1), block(64);
    if (act_dtype == SA_F32)
      hipLaunchKernelGGL(delta_prepare_kernel<float>, grid, block, 0, stream, (const float*)z, zs, conv_w, state,
                         (size_t)state_stride, conv_off, ba, A_log, dt_bias, seg_of_token, cu_q, state_slots, qn, kn,
                         vc, beta, decay, H, Hk, dk, dv, taps);
    else if (act_dtype == SA_BF16)
      hipLaunchKernelGGL(delta_prepare_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)z, zs, conv_w, state,
                         (size_t)state_stride, conv_off, ba, A_log, dt_bias, seg_of_token, cu_q, state_slots, qn, kn,
                         vc, beta, decay, H, Hk, dk, dv, taps);
    else return SA_ERR_UNSUPPORTED;
    SA_LAUNCH_CHECK();
  }
  if (taps > 1) {
    dim3 grid(B, (C + 255) / 256), block(256);
    if (act_dtype == SA_F32)
      hipLaunchKernelGGL(delta_conv_state_kernel<float>, grid, block, 0, stream, (const float*)z, zs, state,
                         (size_t)state_stride, conv_off, cu_q, state_slots, C, taps);
    else
      hipLaunchKernelGGL(delta_conv_state_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)z, zs, state,
                         (size_t)state_stride, conv_off, cu_q, state_slots, C, taps);
    SA_LAUNCH_CHECK();
  }
  if (max_q_len < 8) {
    // single tokens (and portions of a few): 16 columns a wave
    const int waves = dv >= 64 ? 4 : (dv + 15) / 16;
    const int cols = 16 * waves;
    dim3 grid((dv + cols - 1) / cols, H, B), block(64 * waves);
#define GO(RPT)                                                                                                 \
  hipLaunchKernelGGL((delta_recurrence_kernel<RPT, 4, 16>), grid, block, 0, stream, qn, kn, vc, beta, decay,    \
                     state, (size_t)state_stride, cu_q, state_slots, o, H, Hk, dk, dv)
    if (dk <= 64) GO(16);
    else if (dk <= 128) GO(32);
    else GO(64);
#undef GO
    SA_LAUNCH_CHECK();
  } else {
    // prompt portions: 4 columns a wave, four tokens a pass over the state
    const int waves = dv >= 16 ? 4 : (dv + 3) / 4;
    const int cols = 4 * waves;
    dim3 grid((dv + cols - 1) / cols, H, B), block(64 * waves);
#define GO(RPT)                                                                                                 \
  hipLaunchKernelGGL((delta_recurrence_block_kernel<RPT, 32>), grid, block, 0, stream, qn, kn, vc, beta, decay, \
                     state, (size_t)state_stride, cu_q, state_slots, o, H, Hk, dk, dv)
    if (dk <= 64) GO(4);
    else if (dk <= 128) GO(8);
    else GO(16);
#undef GO
    SA_LAUNCH_CHECK();
  }
  {
    const long long TH = (long long)T * H;
    if (TH > 0x7fffffffLL) return SA_ERR_ARG;
    dim3 grid((unsigned)((TH + 3) / 4)), block(256);
    if (act_dtype == SA_F32)
      hipLaunchKernelGGL(delta_gated_norm_kernel<float>, grid, block, 0, stream, o, (const float*)z, zs, C, norm_w,
                         (float*)y, eps, (int)TH, H, dv);
    else
      hipLaunchKernelGGL(delta_gated_norm_kernel<bf16_t>, grid, block, 0, stream, o, (const bf16_t*)z, zs, C, norm_w,
                         (bf16_t*)y, eps, (int)TH, H, dv);
    SA_LAUNCH_CHECK();
  }
  return 0;
}
