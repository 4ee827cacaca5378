// Mixers that carry a state of fixed size from token to token instead of a cache of keys: a linear attention
// with a decay per head, and an element-wise gated recurrence. States live in float32 in slots,
// state[slot][...], one slot a sequence (state_slots[s]); a step reads the state its sequence's earlier tokens left,
// runs the sequence's new rows query_start[s] .. query_start[s+1]-1 in order and writes the state back. What a
// token's output is depends on the tokens before it only, not on how they were cut into steps, beyond rounding.
//
// A sequence's tokens are a dependent chain, so a step of single tokens (or short portions) walks each sequence in
// one go (pass 0). A long portion would leave the GPU to a handful of waves; it is cut into chunks of rows
// instead (items = (sequence, first row, one past the last row), listed in the order of the rows) and run in three
// launches, all chunks side by side: pass 1 runs every chunk from a zero state and keeps what it ends with; the
// combine kernel walks a sequence's chunks in order, S <- A_chunk S + L_chunk, leaving every chunk the state it
// starts from and the slot the state after the last; pass 3 runs every chunk again from its true starting state
// and writes the outputs. Both recurrences are linear in the state, which is all this needs.
//
// All arithmetic is float32 (sums of products with fmaf in a fixed order); inputs are the float32 sums of the
// projections, activations are applied here.
#include "common.h"

#include <math.h>

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

// ------------------------------------------------------ decayed linear attention
// Per head: S_t = decay * S_(t-1) + k_t v_t^T (S is [d][e]), o_t = S_t^T q_t, with q, k, v = act(projection) where
// act is SiLU (activation 1) or nothing (0). Row t of `proj` holds [q (H*d) | k (H*d) | v (H*e) | ...], head by head.
//
// A workgroup of four waves owns 64 value columns of one (sequence, head): a lane is a column, and wave w holds
// the state's rows w * DPT .. w * DPT + DPT - 1 of that column in registers (DPT = a quarter of d, rounded up).
// A token then needs, per wave, the DPT keys and queries of its rows - the same for all 64 lanes - and each lane's
// own value: lane l fetches key and query l (and l + 64, where a wave has more than 64 rows) of the wave's rows from LDS (no
// two lanes the same word), and the update st[i] = decay st[i] + k_i v and the output o += st[i] q_i take k_i and q_i from lane i by a
// lane read into a scalar register, so a token costs a lane 3 DPT arithmetic instructions and no shuffles. The
// waves' partial outputs (over their rows) of SCAN_TOKENS tokens meet in LDS and are added in the order of the waves.
// Keys, queries and the 64 value columns of SCAN_TOKENS tokens at a time are activated once by the workgroup's
// threads on their way into LDS, and the loads of the next tokens are in flight while the current ones are
// computed: a sequence's tokens are a dependent chain, and the only way to be fast along it is to make a token
// cheap and never wait for memory inside it.
// PASS: 0 whole sequences from and to their slots; 1 and 3 the chunks of long portions.
#define SCAN_TOKENS 8
#define SCAN_MAX_D 512

__device__ __forceinline__ float lane_value(float x, int lane) {       // lane: a constant after unrolling
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

template <int DPT, int PASS>
__global__ __launch_bounds__(256) void decay_attention_scan_kernel(
    const float* __restrict__ proj, int row, float* __restrict__ out, float* __restrict__ state,
    const int* __restrict__ query_start, const int* __restrict__ state_slots, const float* __restrict__ decay,
    int H, int d, int e, int activation, const int* __restrict__ items, float* __restrict__ chunk_states) {
  constexpr int MAX_D = 4 * DPT;                        // the keys (and queries) the four waves' rows cover
  constexpr int SCAN_ROW = 2 * MAX_D + 64;              // keys, queries, 64 value columns of a token
  constexpr int SCAN_STAGE_REGS = (SCAN_TOKENS * SCAN_ROW + 255) / 256;
  __shared__ __attribute__((aligned(16))) float kqv_s[SCAN_TOKENS][SCAN_ROW];
  __shared__ float o_s[SCAN_TOKENS][4][64];
  const int wave = threadIdx.x / TIE_WAVE, lane = threadIdx.x & (TIE_WAVE - 1);
  const int h = blockIdx.y;
  const int s = PASS == 0 ? static_cast<int>(blockIdx.z) : items[blockIdx.z * 3];
  const int v_first = blockIdx.x * 64;                  // the workgroup's value columns
  const int v_count = min(64, e - v_first);
  const int col = v_first + lane;
  const bool live = lane < v_count;
  const int d0 = wave * DPT;                            // this wave's rows of the state: d0 .. d0 + DPT - 1 (< d)
  const float lam = decay[h];
  float* S = PASS == 0 ? state + ((static_cast<size_t>(state_slots[s]) * H + h) * d) * e
                       : chunk_states + ((static_cast<size_t>(blockIdx.z) * H + h) * d) * e;
  float st[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i)
    st[i] = (PASS != 1 && live && d0 + i < d) ? S[static_cast<size_t>(d0 + i) * e + col] : 0.f;

  const int t0 = PASS == 0 ? query_start[s] : items[blockIdx.z * 3 + 1];
  const int t1 = PASS == 0 ? query_start[s + 1] : items[blockIdx.z * 3 + 2];
  const size_t q_col = static_cast<size_t>(h) * d, k_col = static_cast<size_t>(H) * d + static_cast<size_t>(h) * d;
  const size_t v_col = 2 * static_cast<size_t>(H) * d + static_cast<size_t>(h) * e;
  // What the workgroup stages of one token: d keys, d queries (not in pass 1, which forms no outputs), and its
  // value columns; value j of these lies at some column of the token's row and at some place of the LDS row.
  const int nq = PASS == 1 ? 0 : d;
  const int per_token = d + nq + v_count;
  float regs[SCAN_STAGE_REGS];
  auto fetch = [&](int tb) {
    const int total = min(SCAN_TOKENS, t1 - tb) * per_token;
#pragma unroll
    for (int r = 0; r < SCAN_STAGE_REGS; ++r) {
      const int idx = threadIdx.x + r * 256;
      regs[r] = 0.f;
      if (idx < total) {
        const int tok = idx / per_token, j = idx - tok * per_token;
        const size_t c = j < d ? k_col + j : (j < d + nq ? q_col + (j - d) : v_col + v_first + (j - d - nq));
        regs[r] = proj[static_cast<size_t>(tb + tok) * row + c];
      }
    }
  };
  auto publish = [&](int tb) {
    const int total = min(SCAN_TOKENS, t1 - tb) * per_token;
#pragma unroll
    for (int r = 0; r < SCAN_STAGE_REGS; ++r) {
      const int idx = threadIdx.x + r * 256;
      if (idx < total) {
        const int tok = idx / per_token, j = idx - tok * per_token;
        const int place = j < d ? j : (j < d + nq ? MAX_D + (j - d) : 2 * MAX_D + (j - d - nq));
        kqv_s[tok][place] = activation ? silu_f(regs[r]) : regs[r];
      }
    }
  };
  constexpr int PER_LANE = (DPT + TIE_WAVE - 1) / TIE_WAVE;   // rows of the wave whose key and query a lane fetches
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += SCAN_TOKENS) {       // uniform for the workgroup
    const int count = min(SCAN_TOKENS, t1 - tb);
    publish(tb);
    __syncthreads();
    if (tb + SCAN_TOKENS < t1) fetch(tb + SCAN_TOKENS); // in flight during the arithmetic below
    for (int tok = 0; tok < count; ++tok) {
      const float v = live ? kqv_s[tok][2 * MAX_D + lane] : 0.f;
      float k_mine[PER_LANE], q_mine[PER_LANE];
#pragma unroll
      for (int g = 0; g < PER_LANE; ++g) {
        const int r = g * TIE_WAVE + lane;
        const bool has_row = r < DPT && d0 + r < d;
        k_mine[g] = has_row ? kqv_s[tok][d0 + r] : 0.f;
        q_mine[g] = (PASS != 1 && has_row) ? kqv_s[tok][MAX_D + d0 + r] : 0.f;
      }
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DPT; ++i) {
        st[i] = fmaf(lam, st[i], lane_value(k_mine[i / TIE_WAVE], i % TIE_WAVE) * v);
        if (PASS != 1) o = fmaf(st[i], lane_value(q_mine[i / TIE_WAVE], i % TIE_WAVE), o);
      }
      if (PASS != 1) o_s[tok][wave][lane] = o;
    }
    __syncthreads();                                    // the next tokens overwrite what was just read
    if (PASS != 1) {
      for (int j = threadIdx.x; j < count * 64; j += 256) {
        const int tok = j >> 6, c = j & 63;
        if (c < v_count)
          out[(static_cast<size_t>(tb + tok) * H + h) * e + v_first + c] =
              ((o_s[tok][0][c] + o_s[tok][1][c]) + o_s[tok][2][c]) + o_s[tok][3][c];
      }
    }
  }
  if (PASS == 3) return;
#pragma unroll
  for (int i = 0; i < DPT; ++i)
    if (live && d0 + i < d) S[static_cast<size_t>(d0 + i) * e + col] = st[i];
}

// Pass 1 on the matrix cores, in float32: what a chunk of n <= 64 tokens ends with from zero is one product,
//   L = sum_j decay^(n-1-j) k_j v_j^T = Kd^T V,   Kd[j] = decay^(n-1-j) k_j,
// and v_mfma_f32_32x32x2_f32 multiplies float32 operands exactly as the scan's fused multiply-adds do (no 16-bit
// rounding of keys, values or decays; the sums differ from the scan's in their order only). A workgroup of four
// waves owns a block of 128 rows x 128 columns of one (chunk, head)'s state: the chunk's keys (activated, times their
// decay) and values (activated) of the block are staged once in LDS, [64 tokens][128], and wave w forms the rows
// 32 w .. 32 w + 31 of four column tiles of 32, two tokens an instruction: lane l hands the instruction key
// (token 2 s + l / 32, row l % 32) and value (token 2 s + l / 32, column l % 32), consecutive lanes consecutive words.
// The accumulators hold, in lane l, column l % 32 and the rows 8 (r / 4) + 4 (l / 32) + r % 4 of register r.
typedef float scan_f16_t __attribute__((ext_vector_type(16)));
#define CHUNK_TOKENS 64
__global__ __launch_bounds__(256) void decay_attention_chunk_state_kernel(
    const float* __restrict__ proj, int row, const float* __restrict__ decay, int H, int d, int e, int activation,
    const int* __restrict__ items, float* __restrict__ chunk_states, int e_blocks) {
  __shared__ float k_s[CHUNK_TOKENS][128];
  __shared__ float v_s[CHUNK_TOKENS][128];
  const int wave = threadIdx.x / TIE_WAVE, lane = threadIdx.x & (TIE_WAVE - 1);
  const int h = blockIdx.y, item = blockIdx.z;
  const int d_first = (blockIdx.x / e_blocks) * 128, e_first = (blockIdx.x % e_blocks) * 128;
  const int t0 = items[item * 3 + 1];
  const int n = items[item * 3 + 2] - t0;               // 1 .. CHUNK_TOKENS (the caller's chunks are no longer)
  const float lam = decay[h];
  const size_t k_col = static_cast<size_t>(H) * d + static_cast<size_t>(h) * d + d_first;
  const size_t v_col = 2 * static_cast<size_t>(H) * d + static_cast<size_t>(h) * e + e_first;
  // decay^m as 2^(m log2 decay): one logarithm a thread (m = 0 apart, so that a decay of zero gives 1, then 0).
  const float log2_lam = log2f(lam);
  constexpr int AHEAD = 8;                              // loads asked for before the first of them is used
  for (int base = threadIdx.x; base < CHUNK_TOKENS * 128; base += 256 * AHEAD) {
    float kr[AHEAD], vr[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int idx = base + u * 256, j = idx >> 7, i = idx & 127;
      const float* r = proj + static_cast<size_t>(t0 + min(j, n - 1)) * row;
      kr[u] = (j < n && d_first + i < d) ? r[k_col + i] : 0.f;
      vr[u] = (j < n && e_first + i < e) ? r[v_col + i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int idx = base + u * 256, j = idx >> 7, i = idx & 127;
      float k = kr[u], v = vr[u];
      if (activation) {
        k = silu_f(k);
        v = silu_f(v);
      }
      const int m = n - 1 - j;
      if (m > 0) k *= exp2f(static_cast<float>(m) * log2_lam);
      k_s[j][i] = j < n ? k : 0.f;
      v_s[j][i] = j < n ? v : 0.f;
    }
  }
  __syncthreads();
  scan_f16_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  const int steps = (n + 1) / 2;                         // a token beyond the chunk is a row of zeros
  const int half = lane >> 5, l32 = lane & 31;
  for (int st = 0; st < steps; ++st) {
    const int j = 2 * st + half;
    const float a = k_s[j][wave * 32 + l32];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, v_s[j][c * 32 + l32], acc[c], 0, 0, 0);
  }
  float* S = chunk_states + ((static_cast<size_t>(item) * H + h) * d) * e;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int col = e_first + c * 32 + l32;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int rw = d_first + wave * 32 + 8 * (r / 4) + 4 * half + (r % 4);
      if (rw < d && col < e) S[static_cast<size_t>(rw) * e + col] = acc[c][r];
    }
  }
}

// Pass 3 on the matrix cores, in float32, for keys of up to 128 dimensions: the outputs of a chunk of n <= 64 tokens
// that starts from the state S are
//   O = diag(decay^(i+1)) (Q S)  +  ((Q K^T) (.) D) V,    D[i][j] = decay^(i-j) for j <= i, else 0,
// three products. A workgroup of four waves owns 128 value columns of one (chunk, head), 64 at a time. Staged in LDS: the chunk's
// queries and keys (activated; rows of 129 words, so that 32 lanes reading one dimension of 32 tokens meet 32 banks),
// its values of the 64 columns, and the starting state's 64 columns. Wave w first forms the 32 x 32 tile
// (w / 2, w % 2) of Q K^T (the tile above the diagonal is not computed), applies D in float32 and leaves it in LDS;
// then the tile (w / 2, w % 2) of O: Q S over the key dimensions, its rows scaled by decay^(i+1), plus P V over the
// chunk's tokens. Operands and sums are float32 throughout; nothing of the state passes through 16 bits.
#define P3_ROW 129
#define P3_FLOATS (2 * CHUNK_TOKENS * P3_ROW + CHUNK_TOKENS * 64 + 128 * 64 + CHUNK_TOKENS * 65)
__global__ __launch_bounds__(256) void decay_attention_chunk_output_kernel(
    const float* __restrict__ proj, int row, float* __restrict__ out, const float* __restrict__ decay, int H, int d,
    int e, int activation, const int* __restrict__ items, const float* __restrict__ chunk_states) {
  extern __shared__ __attribute__((aligned(16))) float p3_smem[];
  float* q_s = p3_smem;                                   // [64][129]
  float* k_s = q_s + CHUNK_TOKENS * P3_ROW;               // [64][129]
  float* v_s = k_s + CHUNK_TOKENS * P3_ROW;               // [64][64]
  float* s_s = v_s + CHUNK_TOKENS * 64;                   // [128][64]
  float* p_s = s_s + 128 * 64;                            // [64][65]
  const int wave = threadIdx.x / TIE_WAVE, lane = threadIdx.x & (TIE_WAVE - 1);
  const int half = lane >> 5, l32 = lane & 31;
  const int h = blockIdx.y, item = blockIdx.z;
  const int t0 = items[item * 3 + 1];
  const int n = items[item * 3 + 2] - t0;
  const float lam = decay[h];
  const float log2_lam = log2f(lam);
  auto power = [&](int m) { return m > 0 ? exp2f(static_cast<float>(m) * log2_lam) : 1.f; };
  const size_t q_col = static_cast<size_t>(h) * d, k_col = static_cast<size_t>(H) * d + static_cast<size_t>(h) * d;
  const size_t v_col = 2 * static_cast<size_t>(H) * d + static_cast<size_t>(h) * e;
  constexpr int AHEAD = 32;                             // every load of a stage in flight at once
  // queries and keys: [token][dimension], 64 x 128 each
  for (int base = threadIdx.x; base < CHUNK_TOKENS * 128; base += 256 * AHEAD) {
    float qr[AHEAD], kr[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int idx = base + u * 256, j = idx >> 7, i = idx & 127;
      const float* r = proj + static_cast<size_t>(t0 + min(j, n - 1)) * row;
      const bool has = j < n && i < d;
      qr[u] = has ? r[q_col + i] : 0.f;
      kr[u] = has ? r[k_col + i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int idx = base + u * 256, j = idx >> 7, i = idx & 127;
      q_s[j * P3_ROW + i] = activation ? silu_f(qr[u]) : qr[u];
      k_s[j * P3_ROW + i] = activation ? silu_f(kr[u]) : kr[u];
    }
  }
  // A workgroup takes two blocks of 64 value columns in turn: the score tile P is formed once. Per block, values
  // [token][column] and the starting state [dimension][column] are asked for (32 of each a thread) ahead of the
  // arithmetic that precedes their use - the score product for the first block, the first block's outputs for the
  // second - and stored to LDS behind it.
  constexpr int EACH = 128 * 64 / 256;
  float vr[EACH], sr[EACH];
  auto fetch = [&](int e_first) {
    const float* S = chunk_states + ((static_cast<size_t>(item) * H + h) * d) * e + e_first;
#pragma unroll
    for (int u = 0; u < EACH; ++u) {
      const int idx = threadIdx.x + u * 256, j = idx >> 6, c = idx & 63;
      const bool col_ok = e_first + c < e;
      vr[u] = (col_ok && j < n) ? proj[static_cast<size_t>(t0 + j) * row + v_col + e_first + c] : 0.f;
      sr[u] = (col_ok && j < d) ? S[static_cast<size_t>(j) * e + c] : 0.f;
    }
  };
  auto publish = [&]() {
#pragma unroll
    for (int u = 0; u < EACH; ++u) {
      const int idx = threadIdx.x + u * 256, j = idx >> 6, c = idx & 63;
      if (j < CHUNK_TOKENS) v_s[j * 64 + c] = activation ? silu_f(vr[u]) : vr[u];
      s_s[j * 64 + c] = sr[u];
    }
  };
  const int e_begin = blockIdx.x * 128, e_end = min(e, e_begin + 128);
  fetch(e_begin);
  __syncthreads();

  const int mt = wave >> 1, ct = wave & 1;              // this wave's tile of rows (tokens) and of columns
  const int d_steps = (min(d, 128) + 1) / 2;
  scan_f16_t acc;
  // P = (Q K^T) (.) D: tile (mt, ct) of the chunk's 64 x 64 scores; nothing above the diagonal
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  if (ct <= mt) {
    for (int st = 0; st < d_steps; ++st) {
      const int kk = 2 * st + half;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(q_s[(mt * 32 + l32) * P3_ROW + kk], k_s[(ct * 32 + l32) * P3_ROW + kk],
                                                 acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int i = mt * 32 + 8 * (r / 4) + 4 * half + (r % 4), j = ct * 32 + l32;
    p_s[i * 65 + j] = (ct <= mt && j <= i && i < n) ? acc[r] * power(i - j) : 0.f;
  }

  for (int e_first = e_begin; e_first < e_end; e_first += 64) {     // uniform for the workgroup
    publish();
    __syncthreads();
    if (e_first + 64 < e_end) fetch(e_first + 64);       // on their way during this block's products
    // O tile (mt, ct): rows scaled Q S, then P V
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    for (int st = 0; st < d_steps; ++st) {
      const int kk = 2 * st + half;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(q_s[(mt * 32 + l32) * P3_ROW + kk], s_s[kk * 64 + ct * 32 + l32], acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] *= power(mt * 32 + 8 * (r / 4) + 4 * half + (r % 4) + 1);
    const int t_steps = (min(n, (mt + 1) * 32) + 1) / 2;   // keys beyond the tile's last row weigh nothing
    for (int st = 0; st < t_steps; ++st) {
      const int kk = 2 * st + half;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(p_s[(mt * 32 + l32) * 65 + kk], v_s[kk * 64 + ct * 32 + l32], acc, 0, 0, 0);
    }
    const int col = e_first + ct * 32 + l32;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = mt * 32 + 8 * (r / 4) + 4 * half + (r % 4);
      if (i < n && col < e) out[(static_cast<size_t>(t0 + i) * H + h) * e + col] = acc[r];
    }
    __syncthreads();                                     // the next block's values and state overwrite these
  }
}

// The chunks of every sequence in order: chunk_states[c] holds what chunk c ends with when started from zero (L)
// and receives the state it really starts from; the slot receives the state after the sequence's last chunk.
// first_item[s] .. first_item[s + 1] - 1 are sequence s's items. One thread an element of the state.
__global__ void decay_attention_combine_kernel(float* __restrict__ chunk_states, float* __restrict__ state,
                                               const int* __restrict__ items, const int* __restrict__ first_item,
                                               const int* __restrict__ state_slots,
                                               const float* __restrict__ decay, int H, int per_head) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t per_state = static_cast<size_t>(H) * per_head;
  if (idx >= per_state) return;
  const int s = blockIdx.y;
  const float lam = decay[idx / per_head];
  float* slot = state + static_cast<size_t>(state_slots[s]) * per_state + idx;
  float S = *slot;
  constexpr int AHEAD = 8;                              // chunks whose values are asked for before the chain needs them
  const int last = first_item[s + 1];
  for (int c0 = first_item[s]; c0 < last; c0 += AHEAD) {
    float local[AHEAD], keep[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int c = min(c0 + u, last - 1);
      local[u] = chunk_states[static_cast<size_t>(c) * per_state + idx];
      keep[u] = powf(lam, static_cast<float>(items[c * 3 + 2] - items[c * 3 + 1]));
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      if (c0 + u >= last) break;
      chunk_states[static_cast<size_t>(c0 + u) * per_state + idx] = S;
      S = fmaf(keep[u], S, local[u]);
    }
  }
  *slot = S;
}

// num_items = 0: every sequence in one go. Otherwise items [num_items][3] = (sequence, first row, one past the last
// row) in the order of the rows, first_item [S + 1] the sequences' ranges of items, and chunk_states
// [num_items][H][d][e] scratch memory: the three launches described at the top.
extern "C" int tie_decay_attention_scan(const float* proj, int row, float* out, float* state, const int* query_start,
                                        const int* state_slots, const float* decay, int S, int H, int d, int e,
                                        int activation, const int* items, const int* first_item, int num_items,
                                        float* chunk_states, int max_chunk_rows, hipStream_t stream) {
  if (S <= 0 || S > 65535 || H <= 0 || H > 65535 || d <= 0 || d > SCAN_MAX_D || e <= 0 || row < 2 * H * d + H * e ||
      num_items < 0 || num_items > 65535 ||
      (num_items > 0 && (items == nullptr || first_item == nullptr || chunk_states == nullptr)))
    return TIE_BAD_ARGUMENT;
  const int col_blocks = (e + 63) / 64;
  const int per = (d + 3) / 4;
  // The chunks' states from zero as one float32 matrix product a block, where the chunks are at most 64 rows long
  // and a state is large enough for blocks of 128 x 128 not to be mostly padding.
  const bool matrix_pass1 = max_chunk_rows > 0 && max_chunk_rows <= CHUNK_TOKENS && d * e >= 32 * 32;
  bool matrix_pass3 = matrix_pass1 && d <= 128;          // the outputs likewise, for keys of up to 128 dimensions
  if (matrix_pass3) {
    static bool configured = false;                      // more LDS than a kernel gets unasked
    if (!configured) {
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&decay_attention_chunk_output_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 static_cast<int>(P3_FLOATS * sizeof(float)));
      if (err != hipSuccess) return static_cast<int>(err);
      configured = true;
    }
  }
#define LAUNCH_PASS(DPT, PASS, COUNT)                                                                \
  decay_attention_scan_kernel<DPT, PASS><<<dim3(col_blocks, H, COUNT), 256, 0, stream>>>(         \
      proj, row, out, state, query_start, state_slots, decay, H, d, e, activation, items, chunk_states)
#define LAUNCH(DPT)                                                                                  \
  {                                                                                                  \
    if (num_items == 0) {                                                                            \
      LAUNCH_PASS(DPT, 0, S);                                                                        \
    } else {                                                                                         \
      if (matrix_pass1) {                                                                            \
        const int e_blocks = (e + 127) / 128, d_blocks = (d + 127) / 128;                            \
        decay_attention_chunk_state_kernel<<<dim3(d_blocks * e_blocks, H, num_items), 256, 0, stream>>>( \
            proj, row, decay, H, d, e, activation, items, chunk_states, e_blocks);                   \
      } else {                                                                                       \
        LAUNCH_PASS(DPT, 1, num_items);                                                              \
      }                                                                                              \
      const size_t per_state = static_cast<size_t>(H) * d * e;                                       \
      decay_attention_combine_kernel<<<dim3(static_cast<unsigned>((per_state + 255) / 256), S), 256, 0, stream>>>( \
          chunk_states, state, items, first_item, state_slots, decay, H, d * e);                     \
      if (matrix_pass3) {                                                                            \
        decay_attention_chunk_output_kernel<<<dim3((e + 127) / 128, H, num_items), 256, P3_FLOATS * sizeof(float), stream>>>( \
            proj, row, out, decay, H, d, e, activation, items, chunk_states);                        \
      } else {                                                                                       \
        LAUNCH_PASS(DPT, 3, num_items);                                                              \
      }                                                                                              \
    }                                                                                                \
  }
  if (per <= 8) LAUNCH(8)
  else if (per <= 16) LAUNCH(16)
  else if (per <= 32) LAUNCH(32)
  else if (per <= 64) LAUNCH(64)
  else LAUNCH(128)
#undef LAUNCH
#undef LAUNCH_PASS
  return tie_launch_status();
}

// --------------------------------------------------- gated norm of the heads' outputs
// out[t] = RMSNorm(o[t]) * w * sigmoid(gate[t]) over rows of n values (all heads side by side); gate rows are
// gate_row floats apart (a view into the projection's rows). Statistics in float32.
template <typename TO>
__global__ void gated_rms_norm_kernel(const float* __restrict__ o, const float* __restrict__ w, float eps,
                                      const float* __restrict__ gate, int gate_row, TO* __restrict__ out, int n) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const float* r = o + t * n;
  const float* g = gate + t * gate_row;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) ss = fmaf(r[c], r[c], ss);
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    store_from_float(out + t * n + c, (r[c] * inv) * w[c] * sigmoid_f(g[c]));
}

extern "C" int tie_gated_rms_norm(const float* o, const float* w, float eps, const float* gate, int gate_row, void* out,
                                  int out_dtype, int T, int n, hipStream_t stream) {
  if (T <= 0 || n <= 0 || gate_row < n) return TIE_BAD_ARGUMENT;
  const int threads = n >= 2048 ? 512 : (n >= 512 ? 256 : 64);
  if (out_dtype == TIE_F32)
    gated_rms_norm_kernel<float><<<T, threads, 0, stream>>>(o, w, eps, gate, gate_row, static_cast<float*>(out), n);
  else if (out_dtype == TIE_BF16)
    gated_rms_norm_kernel<bf16_t><<<T, threads, 0, stream>>>(o, w, eps, gate, gate_row, static_cast<bf16_t*>(out), n);
  else
    return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}

// ------------------------------------------------------------- minimal gated recurrent unit
// Element by element: z = sigmoid(a), c = candidate(u) = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
// S_t = (1 - z) S_(t-1) + z c, out_t = S_t * silu(g). Row t of `proj` holds [a (n) | u (n) | g (n)]; `bias` (or
// null) holds 3 n values that are added to them here, so that the projection needs no pass of its own for them.
// A thread owns one channel of one sequence and walks its rows; neighbouring threads read neighbouring floats.
// Chunks (see the top): pass 1 leaves a chunk's product of (1 - z) in chunk_a and what it ends with from zero in
// chunk_b; the combine kernel turns chunk_b into the state each chunk starts from; pass 3 writes the outputs.
template <typename TO, int PASS>
__global__ void min_gru_scan_kernel(const float* __restrict__ proj, int row, TO* __restrict__ out,
                                    float* __restrict__ state, const int* __restrict__ query_start,
                                    const int* __restrict__ state_slots, int n, const int* __restrict__ items,
                                    float* __restrict__ chunk_a, float* __restrict__ chunk_b,
                                    const float* __restrict__ bias) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const float ba = bias ? bias[c] : 0.f, bu = bias ? bias[n + c] : 0.f, bg = bias ? bias[2 * n + c] : 0.f;
  const int s = PASS == 0 ? static_cast<int>(blockIdx.y) : items[blockIdx.y * 3];
  float* sp = PASS == 0 ? state + static_cast<size_t>(state_slots[s]) * n + c
                        : chunk_b + static_cast<size_t>(blockIdx.y) * n + c;
  float st = PASS == 1 ? 0.f : *sp;
  float keep = 1.f;
  const int t0 = PASS == 0 ? query_start[s] : items[blockIdx.y * 3 + 1];
  const int t1 = PASS == 0 ? query_start[s + 1] : items[blockIdx.y * 3 + 2];
  // Eight tokens' values are asked for before the first of them is used: the chain through the state is short
  // arithmetic, and what it would otherwise wait for, token after token, is memory.
  constexpr int AHEAD = 8;
  for (int t = t0; t < t1; t += AHEAD) {
    float a[AHEAD], u[AHEAD], g[AHEAD];
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {
      const float* r = proj + static_cast<size_t>(min(t + j, t1 - 1)) * row + c;
      a[j] = r[0];
      u[j] = r[n];
      g[j] = PASS == 1 ? 0.f : r[2 * static_cast<size_t>(n)];
    }
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {
      if (t + j >= t1) break;
      const float z = sigmoid_f(a[j] + ba);
      const float x = u[j] + bu;
      const float cand = x >= 0.f ? x + 0.5f : sigmoid_f(x);
      st = fmaf(z, cand, (1.0f - z) * st);
      if (PASS == 1) keep *= 1.0f - z;
      else store_from_float(out + static_cast<size_t>(t + j) * n + c, st * silu_f(g[j] + bg));
    }
  }
  if (PASS == 3) return;
  *sp = st;
  if (PASS == 1) chunk_a[static_cast<size_t>(blockIdx.y) * n + c] = keep;
}

__global__ void min_gru_combine_kernel(const float* __restrict__ chunk_a, float* __restrict__ chunk_b,
                                       float* __restrict__ state, const int* __restrict__ first_item,
                                       const int* __restrict__ state_slots, int n) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const int s = blockIdx.y;
  float* slot = state + static_cast<size_t>(state_slots[s]) * n + c;
  float S = *slot;
  for (int i = first_item[s]; i < first_item[s + 1]; ++i) {
    const float local = chunk_b[static_cast<size_t>(i) * n + c];
    chunk_b[static_cast<size_t>(i) * n + c] = S;
    S = fmaf(chunk_a[static_cast<size_t>(i) * n + c], S, local);
  }
  *slot = S;
}

// num_items = 0: every sequence in one go; otherwise items, first_item as for the linear attention and chunk_ab
// [2][num_items][n] scratch memory.
extern "C" int tie_min_gru_scan(const float* proj, int row, void* out, int out_dtype, float* state,
                                const int* query_start, const int* state_slots, int S, int n, const int* items,
                                const int* first_item, int num_items, float* chunk_ab, const float* bias,
                                hipStream_t stream) {
  if (S <= 0 || S > 65535 || n <= 0 || row < 3 * n || num_items < 0 || num_items > 65535 ||
      (num_items > 0 && (items == nullptr || first_item == nullptr || chunk_ab == nullptr)) ||
      (out_dtype != TIE_F32 && out_dtype != TIE_BF16))
    return TIE_BAD_ARGUMENT;
  const int threads = n >= 256 ? 256 : 64;
  const unsigned across = (n + threads - 1) / threads;
  float* chunk_a = chunk_ab;
  float* chunk_b = chunk_ab == nullptr ? nullptr : chunk_ab + static_cast<size_t>(num_items) * n;
#define LAUNCH_PASS(TO, PASS, COUNT)                                                                              \
  min_gru_scan_kernel<TO, PASS><<<dim3(across, COUNT), threads, 0, stream>>>(                                     \
      proj, row, static_cast<TO*>(out), state, query_start, state_slots, n, items, chunk_a, chunk_b, bias)
#define LAUNCH(TO)                                                                                                \
  {                                                                                                               \
    if (num_items == 0) {                                                                                         \
      LAUNCH_PASS(TO, 0, S);                                                                                      \
    } else {                                                                                                      \
      LAUNCH_PASS(TO, 1, num_items);                                                                              \
      min_gru_combine_kernel<<<dim3(across, S), threads, 0, stream>>>(chunk_a, chunk_b, state, first_item,        \
                                                                      state_slots, n);                            \
      LAUNCH_PASS(TO, 3, num_items);                                                                              \
    }                                                                                                             \
  }
  if (out_dtype == TIE_F32) LAUNCH(float)
  else LAUNCH(bf16_t)
#undef LAUNCH
#undef LAUNCH_PASS
  return tie_launch_status();
}
