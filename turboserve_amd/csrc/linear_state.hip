// Gated linear attention: a mixer whose memory is one matrix per head and request instead of a
// cache of keys.  Per head, with keys of D and values of Dv elements, the state S [D, Dv] (32-bit,
// zero when a request starts) takes every token as
//
//     S <- diag(a_t) S + k_t v_t^T        o_t = S^T q_t
//
// with a decay a_t in (0, 1) per key channel: a_t = sigmoid(z_t)^(1 / tau), z_t = A2 y_t + b, where
// y_t (a few numbers per token) comes out of the layer's projection like q, k, v and the output gate.
// Everything that enters the recurrence is 32-bit: z, its log-sigmoid, the decay, q / sqrt(D), k, v, S, o.
//
// Row of the projection (type T, or `splits` 32-bit partial sums): [H D q | H D k | H Dv v | H Dv gate | R y].
//
// ts_linear_state_scan walks the tokens of one piece of a request with the state in registers: a
// block of 256 threads owns one head and 64 value columns, thread (column c, quarter p) holds a quarter of
// the rows of S[:, c], one after the other (four rows' staged values are one LDS read).  Eight tokens at a time are staged in LDS (q, k and the decays,
// which the block computes from y), then every thread updates its rows and leaves its share of o;
// the four shares of a column meet in LDS.  Three uses:
//   whole  the piece is all the tokens a request brings; S comes from the request's slot and
//          goes back there.  Single tokens and short portions.
//   long portions are cut into pieces of `piece` tokens that run side by side, in three launches:
//   local  every piece from a zero state, no output: it leaves its own S and the product of its decays;
//   (ts_linear_state_carry walks a request's pieces in order: the state before piece i is the slot's
//          state carried through pieces 0..i-1; it puts that state where the piece's own S stood and
//          leaves the final one in the slot)
//   output every piece again, from the state before it, writing o.
// The recurrence is the same in every use; only the grouping of the sums differs, by rounding.
//
// ts_linear_state_finish: o of each head divided by its root mean square (eps inside the root),
// times a gain [Dv] shared by the heads, times silu(gate), rounded to the run type.
#include "common.hpp"

#define LS_COLS 64      // value columns of a block
#define LS_QUARTERS 4   // threads per column
#define LS_BATCH 8      // tokens staged at a time
#define LS_MAX_DIM 256  // key channels (one thread each computes a channel's decay)
#define LS_MAX_LOW 128  // width of y

typedef float ls_f32x4 __attribute__((ext_vector_type(4)));

// The sum of a projection's partial sums, added in split order, eight loads in flight at a time (a
// loop of load, wait, add would cost a trip to memory per split).
template <typename P>
__device__ __forceinline__ float ls_folded(const P* p, int splits, size_t stride) {
  if (splits == 1) return to_float(p[0]);
  float s = 0.f;
  for (int first = 0; first < splits; first += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = to_float(p[(size_t)min(first + j, splits - 1) * stride]);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (first + j < splits) s += v[j];
  }
  return s;
}

struct LsPiece {
  int seq;    // request of the step
  int first;  // first row
  int count;  // rows
  int pad;
};

// MODE 0: whole (pieces from query_start_loc), 1: local, 2: output.
template <typename T, typename P, int ROWS, int MODE>
__global__ void __launch_bounds__(LS_COLS * LS_QUARTERS)
linear_state_scan_kernel(float* __restrict__ out, const P* __restrict__ proj, int splits, size_t split_stride,
                         const T* __restrict__ a2, const T* __restrict__ a2_bias, float inv_tau,
                         float* __restrict__ state, const int* __restrict__ state_slots,
                         const int* __restrict__ query_start_loc, int first_seq, const LsPiece* __restrict__ pieces,
                         float* __restrict__ piece_state, float* __restrict__ piece_decay, int heads, int dim, int vdim,
                         int low) {
  __shared__ __attribute__((aligned(16))) float qs[LS_BATCH][LS_MAX_DIM];
  __shared__ __attribute__((aligned(16))) float ks[LS_BATCH][LS_MAX_DIM];
  __shared__ __attribute__((aligned(16))) float as[LS_BATCH][LS_MAX_DIM];
  __shared__ float ys[LS_BATCH][LS_MAX_LOW];
  __shared__ float shares[LS_BATCH][LS_QUARTERS][LS_COLS];
  const int item = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int c = tid % LS_COLS, p = tid / LS_COLS;
  const int col = blockIdx.z * LS_COLS + c;
  const bool has_col = col < vdim;
  int seq, first, count;
  if (MODE == 0) {
    seq = first_seq + item;
    first = query_start_loc[seq];
    count = query_start_loc[seq + 1] - first;
  } else {
    seq = pieces[item].seq;
    first = pieces[item].first;
    count = pieces[item].count;
  }
  const size_t width = (size_t)2 * heads * dim + (size_t)2 * heads * vdim + low;
  const size_t q_at = (size_t)h * dim, k_at = (size_t)heads * dim + (size_t)h * dim;
  const size_t v_at = (size_t)2 * heads * dim + (size_t)h * vdim, y_at = (size_t)2 * heads * dim + (size_t)2 * heads * vdim;
  const float q_scale = rsqrtf((float)dim);
  const size_t per_head = (size_t)dim * vdim;

  // The thread's rows of the state: d = p * ROWS + r.
  float s[ROWS];
  const float* from = nullptr;
  if (MODE == 0) from = state + ((size_t)state_slots[seq] * heads + h) * per_head;
  if (MODE == 2) from = piece_state + ((size_t)item * heads + h) * per_head;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = p * ROWS + r;
    s[r] = (from && has_col && d < dim) ? from[(size_t)d * vdim + col] : 0.f;
  }
  // Thread d < dim computes channel d's decay; in local mode it also keeps the product of them.
  float decay_product = 1.f;
  // Channels from dim up to the four quarters' ROWS are read with the others, four at a time: zero keys
  // and queries there, once, so that their rows of the state stay zero and add nothing.
  for (int i = tid; i < LS_BATCH * LS_MAX_DIM; i += blockDim.x) {
    (&qs[0][0])[i] = 0.f;
    (&ks[0][0])[i] = 0.f;
    (&as[0][0])[i] = 0.f;
  }
  for (int i = tid; i < LS_BATCH * LS_MAX_LOW; i += blockDim.x) (&ys[0][0])[i] = 0.f;  // (rows of a short batch are multiplied too)

  for (int base = 0; base < count; base += LS_BATCH) {
    const int n = min(LS_BATCH, count - base);
    __syncthreads();  // the batch before is done with the staged values and the shares
    for (int i = tid; i < n * dim; i += blockDim.x) {
      const int b = i / dim, d = i % dim;
      const P* row = proj + (size_t)(first + base + b) * width;
      if (MODE != 1) qs[b][d] = ls_folded(row + q_at + d, splits, split_stride) * q_scale;
      ks[b][d] = ls_folded(row + k_at + d, splits, split_stride);
    }
    for (int i = tid; i < n * low; i += blockDim.x) {
      const int b = i / low, j = i % low;
      ys[b][j] = ls_folded(proj + (size_t)(first + base + b) * width + y_at + j, splits, split_stride);
    }
    __syncthreads();
    if (tid < dim) {
      const T* w = a2 + ((size_t)h * dim + tid) * low;
      const float bias = to_float(a2_bias[(size_t)h * dim + tid]);
      // The channel's row of A2 is read once per batch, eight elements in flight at a time (read
      // inside the loop over tokens it cost a trip to the caches per token and element).
      float z[LS_BATCH];
#pragma unroll
      for (int b = 0; b < LS_BATCH; ++b) z[b] = bias;
      for (int j0 = 0; j0 < low; j0 += 8) {
        float wv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) wv[u] = j0 + u < low ? to_float(w[j0 + u]) : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int j = min(j0 + u, low - 1);  // past the end: weight 0 on a value that is there
#pragma unroll
          for (int b = 0; b < LS_BATCH; ++b) z[b] = fmaf(wv[u], ys[b][j], z[b]);
        }
      }
#pragma unroll
      for (int b = 0; b < LS_BATCH; ++b) {
        if (b < n) {
          // log sigmoid(z) = min(z, 0) - log(1 + exp(-|z|)); the decay is exp of it over tau.
          const float a = expf((fminf(z[b], 0.f) - log1pf(expf(-fabsf(z[b])))) * inv_tau);
          as[b][tid] = a;
          if (MODE == 1) decay_product *= a;
        }
      }
    }
    __syncthreads();
    float v[LS_BATCH];
#pragma unroll
    for (int b = 0; b < LS_BATCH; ++b)
      v[b] = (b < n && has_col) ? ls_folded(proj + (size_t)(first + base + b) * width + v_at + col, splits, split_stride) : 0.f;
#pragma unroll
    for (int b = 0; b < LS_BATCH; ++b) {
      if (b < n) {
        float o = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          // Four rows' staged values at once (rows beyond the head's channels hold what the batch
          // before left or nothing: their state stays zero because their k is never staged: see below).
          const ls_f32x4 a4 = *reinterpret_cast<const ls_f32x4*>(&as[b][p * ROWS + r]);
          const ls_f32x4 k4 = *reinterpret_cast<const ls_f32x4*>(&ks[b][p * ROWS + r]);
          ls_f32x4 q4 = ls_f32x4{0.f, 0.f, 0.f, 0.f};
          if (MODE != 1) q4 = *reinterpret_cast<const ls_f32x4*>(&qs[b][p * ROWS + r]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            s[r + e] = fmaf(a4[e], s[r + e], k4[e] * v[b]);
            if (MODE != 1) o = fmaf(s[r + e], q4[e], o);
          }
        }
        if (MODE != 1) shares[b][p][c] = o;
      }
    }
    if (MODE != 1) {
      __syncthreads();
      for (int i = tid; i < n * LS_COLS; i += blockDim.x) {
        const int b = i / LS_COLS, cc = i % LS_COLS;
        const int to = blockIdx.z * LS_COLS + cc;
        if (to < vdim)
          out[((size_t)(first + base + b) * heads + h) * vdim + to] =
              (shares[b][0][cc] + shares[b][1][cc]) + (shares[b][2][cc] + shares[b][3][cc]);
      }
    }
  }
  float* to = nullptr;
  if (MODE == 0) to = state + ((size_t)state_slots[seq] * heads + h) * per_head;
  if (MODE == 1) to = piece_state + ((size_t)item * heads + h) * per_head;
  if (to && has_col) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = p * ROWS + r;
      if (d < dim) to[(size_t)d * vdim + col] = s[r];
    }
  }
  if (MODE == 1 && blockIdx.z == 0 && tid < dim) piece_decay[((size_t)item * heads + h) * dim + tid] = decay_product;
}

// One thread per element of a head's state; request `seq` of the list owns pieces first..first+count-1.
struct LsCarry {
  int slot_seq;  // request of the step (its state slot is looked up on the device)
  int first;     // its first piece
  int count;     // its pieces
  int pad;
};

__global__ void linear_state_carry_kernel(float* __restrict__ state, const int* __restrict__ state_slots,
                                          const LsCarry* __restrict__ carries, float* __restrict__ piece_state,
                                          const float* __restrict__ piece_decay, int heads, int dim, int vdim) {
  const LsCarry carry = carries[blockIdx.x];
  const int h = blockIdx.y;
  const size_t per_head = (size_t)dim * vdim;
  const size_t e = (size_t)blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= per_head) return;
  const int d = (int)(e / vdim);
  float* slot = state + ((size_t)state_slots[carry.slot_seq] * heads + h) * per_head + e;
  float s = *slot;
  for (int i = carry.first; i < carry.first + carry.count; ++i) {
    float* own = piece_state + ((size_t)i * heads + h) * per_head + e;
    const float local = *own;
    *own = s;  // the state this piece starts from
    s = fmaf(piece_decay[((size_t)i * heads + h) * dim + d], s, local);
  }
  *slot = s;
}

template <typename T, typename P, int MODE>
static int scan_launch(dim3 grid, hipStream_t stream, float* out, const void* proj, int splits, long split_stride,
                       const void* a2, const void* a2_bias, float inv_tau, float* state, const int* state_slots,
                       const int* query_start_loc, int first_seq, const void* pieces, float* piece_state,
                       float* piece_decay, int heads, int dim, int vdim, int low) {
  const dim3 block(LS_COLS * LS_QUARTERS);
  const int rows = (dim + LS_QUARTERS - 1) / LS_QUARTERS;
#define LS_GO(ROWS)                                                                                                   \
  hipLaunchKernelGGL((linear_state_scan_kernel<T, P, ROWS, MODE>), grid, block, 0, stream, out, (const P*)proj, splits, \
                     (size_t)split_stride, (const T*)a2, (const T*)a2_bias, inv_tau, state, state_slots,              \
                     query_start_loc, first_seq, (const LsPiece*)pieces, piece_state, piece_decay, heads, dim, vdim, low)
  if (rows <= 8) LS_GO(8);
  else if (rows <= 16) LS_GO(16);
  else if (rows <= 32) LS_GO(32);
  else LS_GO(64);
#undef LS_GO
  return ts_launch_status();
}

// mode 0: `items` requests from `first_seq` on, each whole; 1, 2: `items` pieces.
extern "C" int ts_linear_state_scan(float* out, const void* proj, int in_f32, int splits, long split_stride,
                                    const void* a2, const void* a2_bias, float tau, float* state,
                                    const int* state_slots, const int* query_start_loc, int first_seq,
                                    const void* pieces, float* piece_state, float* piece_decay, int items, int heads,
                                    int dim, int vdim, int low, int mode, int dtype, hipStream_t stream) {
  if (items == 0) return TS_OK;
  if (!proj || !a2 || !a2_bias || !(tau > 0.f)) return TS_ERR_ARG;
  if (mode == 0 && (!out || !state || !state_slots || !query_start_loc)) return TS_ERR_ARG;
  if (mode == 1 && (!pieces || !piece_state || !piece_decay)) return TS_ERR_ARG;
  if (mode == 2 && (!out || !pieces || !piece_state)) return TS_ERR_ARG;
  if (mode < 0 || mode > 2) return TS_ERR_ARG;
  if (heads < 1 || heads > 65535 || dim < 1 || dim > LS_MAX_DIM || vdim < 1 || low < 1 || low > LS_MAX_LOW || splits < 1)
    return TS_ERR_SHAPE;
  const dim3 grid(items, heads, (vdim + LS_COLS - 1) / LS_COLS);
  if (grid.z > 65535) return TS_ERR_SHAPE;
  const float inv_tau = 1.f / tau;
#define LS_MODES(T, P, SPLITS, STRIDE)                                                                                  \
  (mode == 0   ? scan_launch<T, P, 0>(grid, stream, out, proj, SPLITS, STRIDE, a2, a2_bias, inv_tau, state, state_slots,  \
                                      query_start_loc, first_seq, pieces, piece_state, piece_decay, heads, dim, vdim, low) \
   : mode == 1 ? scan_launch<T, P, 1>(grid, stream, out, proj, SPLITS, STRIDE, a2, a2_bias, inv_tau, state, state_slots,  \
                                      query_start_loc, first_seq, pieces, piece_state, piece_decay, heads, dim, vdim, low) \
               : scan_launch<T, P, 2>(grid, stream, out, proj, SPLITS, STRIDE, a2, a2_bias, inv_tau, state, state_slots,  \
                                      query_start_loc, first_seq, pieces, piece_state, piece_decay, heads, dim, vdim, low))
  if (dtype == TS_F32) return LS_MODES(float, float, splits, split_stride);
  if (dtype == TS_BF16 && in_f32) return LS_MODES(bf16_t, float, splits, split_stride);
  if (dtype == TS_BF16) return LS_MODES(bf16_t, bf16_t, 1, 0);
#undef LS_MODES
  return TS_ERR_DTYPE;
}

extern "C" int ts_linear_state_carry(float* state, const int* state_slots, const void* carries, float* piece_state,
                                     const float* piece_decay, int requests, int heads, int dim, int vdim,
                                     hipStream_t stream) {
  if (requests == 0) return TS_OK;
  if (!state || !state_slots || !carries || !piece_state || !piece_decay) return TS_ERR_ARG;
  if (heads < 1 || heads > 65535 || dim < 1 || vdim < 1) return TS_ERR_SHAPE;
  const size_t per_head = (size_t)dim * vdim;
  const dim3 grid(requests, heads, (unsigned)((per_head + 255) / 256));
  if (grid.z > 65535) return TS_ERR_SHAPE;
  hipLaunchKernelGGL(linear_state_carry_kernel, grid, dim3(256), 0, stream, state, state_slots, (const LsCarry*)carries,
                     piece_state, piece_decay, heads, dim, vdim);
  return ts_launch_status();
}

// One wavefront per (token, head): o [T, H, Dv] 32-bit, the gate inside the projection's rows.
template <typename T, typename P>
__global__ void __launch_bounds__(256)
linear_state_finish_kernel(T* __restrict__ y, const float* __restrict__ o, const P* __restrict__ proj, int splits,
                           size_t split_stride, const T* __restrict__ gain, float eps, long items, int heads, int dim,
                           int vdim, int low) {
  const long item = (long)blockIdx.x * 4 + threadIdx.x / TS_WAVE;
  const int lane = threadIdx.x % TS_WAVE;
  if (item >= items) return;  // a whole wavefront leaves: the reductions below are per wavefront
  const long t = item / heads;
  const int h = (int)(item % heads);
  const size_t width = (size_t)2 * heads * dim + (size_t)2 * heads * vdim + low;
  const P* gate = proj + (size_t)t * width + (size_t)2 * heads * dim + (size_t)heads * vdim + (size_t)h * vdim;
  const float* row = o + (size_t)item * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += TS_WAVE) ss = fmaf(row[i], row[i], ss);
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)vdim + eps);
  for (int i = lane; i < vdim; i += TS_WAVE) {
    const float g = ls_folded(gate + i, splits, split_stride);
    y[(size_t)item * vdim + i] = from_float<T>(row[i] * r * to_float(gain[i]) * (g / (1.f + expf(-g))));
  }
}

extern "C" int ts_linear_state_finish(void* y, const float* o, const void* proj, int in_f32, int splits,
                                      long split_stride, const void* gain, float eps, int tokens, int heads, int dim,
                                      int vdim, int low, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!y || !o || !proj || !gain) return TS_ERR_ARG;
  if (heads < 1 || dim < 1 || vdim < 1 || low < 0 || splits < 1) return TS_ERR_SHAPE;
  const long items = (long)tokens * heads;
  const dim3 grid((unsigned)((items + 3) / 4)), block(256);
  if (dtype == TS_F32)
    hipLaunchKernelGGL((linear_state_finish_kernel<float, float>), grid, block, 0, stream, (float*)y, o, (const float*)proj, splits, (size_t)split_stride, (const float*)gain, eps, items, heads, dim, vdim, low);
  else if (dtype == TS_BF16 && in_f32)
    hipLaunchKernelGGL((linear_state_finish_kernel<bf16_t, float>), grid, block, 0, stream, (bf16_t*)y, o, (const float*)proj, splits, (size_t)split_stride, (const bf16_t*)gain, eps, items, heads, dim, vdim, low);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((linear_state_finish_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (bf16_t*)y, o, (const bf16_t*)proj, 1, (size_t)0, (const bf16_t*)gain, eps, items, heads, dim, vdim, low);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
