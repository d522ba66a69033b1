// A whole stack of pre-norm layers (norm, attention over the paged cache, norm, dense feed-forward)
// for one decode step of up to 16 sequences, as ONE kernel on gfx950; bfloat16 weights and cache,
// compiled once per head size (-DBT_HEAD_DIM=N).
//
// Why one kernel: a decode step of such a stack is five or six short kernels a layer, each of which
// starts with empty memory pipes, waits a microsecond for its first bytes and drains before the
// next may begin, so that the weights arrive at a third of what HBM delivers.  Here one work-group
// per compute unit stays for the whole stack.  A layer is five phases (norm + fused projection,
// attention, output projection, norm + feed-forward in, feed-forward out) with a barrier across
// the grid between them, and the weights of a phase are asked for one or two phases earlier, into
// registers, so that memory never idles while the work-groups wait for each other.
//
// How the work-groups talk: each XCD has an L2 of its own, so what one work-group writes for the
// others (queries, attention output, hidden activations, the residual stream, and the new keys
// and values) is written and read at device scope (write-through stores, loads that miss the L2:
// relaxed atomic accesses of agent scope), and nothing else is.  The barrier is counters of
// relaxed atomics, one per group of work-groups and one on top, with no fence: a fence would write
// the whole L2 back every time.  Before it signals, every wave waits for its own stores to be
// acknowledged.  All work-groups must be resident at once, so the grid is never larger than the
// number of compute units; a wait that lasts absurdly long sets a flag and gives up, so the kernel
// always ends, and the host reports the flag as an error.
//
// Each product follows the skinny product kernel: the weights are the MFMA's A operand (a lane
// holds eight K values of one output column), the step's rows the B operand, eight waves split K
// and meet in LDS.  A work-group owns the same columns of the residual stream in both products
// that add to it, and keeps them in registers from the first layer to the last.

#include "host.h"
#include "attention_tile.h"
#include "epilogue.h"

typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;

#define STACK_WAVES 8
#define STACK_THREADS (STACK_WAVES * 64)
#define STACK_MAX_ROWS 16
#define STACK_SPIN_LIMIT (1 << 21)
// words of the barrier's memory: [0] top counter, [32 + 32 g] counter of group g, [320] gave up
#define STACK_SYNC_WORDS 512
#define STACK_SYNC_FAILED 320

// A pointer read from memory is a generic one to the compiler, and loads through it would be flat
// loads, which count as LDS traffic too: every wait for LDS would then wait for the weights in
// flight.  The pointers of the table are therefore declared as pointers to global memory.
#define GLOBAL_PTR(T) __attribute__((address_space(1))) T*

// Elements from one layer's place in an exchange buffer to the next: the place's size rounded up to
// whole 256-byte units.
__host__ __device__ inline int64_t stack_place(int64_t elements, int element_bytes) {
  return ((elements * element_bytes + 255) & ~(int64_t)255) / element_bytes;
}

// One layer's tensors (a device array of these is the stack).
struct StackLayer {
  GLOBAL_PTR(const float) norm1_scale;
  GLOBAL_PTR(const float) norm1_shift;   // or null
  GLOBAL_PTR(const float) norm2_scale;
  GLOBAL_PTR(const float) norm2_shift;   // or null
  // The four matrices, packed for this kernel (see Columns): for each group of `cols` output
  // columns, the chunks of 32 K values one after the other, [group][chunk][cols][32], K and the
  // last group padded with zeros.  A wave's load of a chunk is then one contiguous run of bytes and
  // a work-group's matrix one contiguous block, read front to back.
  GLOBAL_PTR(const bf16_t) qkv_weight;   // of [n_q + 2 n_kv][width]
  GLOBAL_PTR(const float) qkv_bias;      // or null
  GLOBAL_PTR(const bf16_t) out_weight;   // of [width][n_q]
  GLOBAL_PTR(const float) out_bias;
  GLOBAL_PTR(const bf16_t) up_weight;    // of [inner][width]
  GLOBAL_PTR(const float) up_bias;
  GLOBAL_PTR(const bf16_t) down_weight;  // of [width][inner]
  GLOBAL_PTR(const float) down_bias;
  GLOBAL_PTR(bf16_t) keys;               // this layer's planes of the paged cache
  GLOBAL_PTR(bf16_t) values;
  float eps1, eps2;
  float scale;                // multiplies q . k
  int reserved;
};

// Mirrored field by field by a ctypes.Structure.
struct StackArgs {
  const StackLayer* layers;
  int n_layers;
  int rows;                   // sequences of the step, one token each
  float* x;                   // [rows][ldx] residual stream, float32, updated in place
  int64_t ldx;
  int width, inner, heads, kv_heads;
  int norm_kind;              // 0 layer norm, 1 RMS norm
  int act;                    // Activation
  int window;
  int max_blocks;
  int cols_qkv, cols_up, cols_x;   // output columns a work-group owns in the fused projection, the feed-forward's
                                   // first product, and the two products that add to the stream (multiples of four)
  const int* blocks;          // [rows][max_blocks]
  const int* positions;       // [rows] position of each sequence's token
  // What the work-groups exchange, a place of its own for every layer: an address is written once
  // in a launch, and read only after that, so readers may take it through their L2.
  // The places are stack_place(...) elements apart and the buffers 256-byte aligned.
  bf16_t* q;                  // [layers] x [rows][heads * head_dim]
  bf16_t* mixed;              // [layers] x [rows][heads * head_dim]
  bf16_t* hidden;             // [layers] x [rows][inner]
  float* between;             // [layers][2] x [rows][width] the residual stream after the mixer / the feed-forward
  unsigned* sync;             // STACK_SYNC_WORDS words, zero at launch
  // null, or [work-groups][STACK_CLOCK_LAYERS][10] 64-bit wall-clock ticks (100 MHz): when each of
  // the first layers' five phases began (the barrier before it had opened) and when its work was done
  unsigned long long* clocks;
};
#define STACK_CLOCK_LAYERS 4

__device__ __forceinline__ float4 load_global_f32x4(GLOBAL_PTR(const float) p) {
  floatx4 v = *(GLOBAL_PTR(const floatx4))p;
  return make_float4(v[0], v[1], v[2], v[3]);
}

// --- what the work-groups exchange ------------------------------------------------------------
// Written through to memory (device scope).  Read with ordinary loads: every address is written
// at most once in a launch and read only after the barrier behind that write, so no L2 can hold
// an older copy of it, and the 32 compute units of an XCD share one fetch.  (Read at device
// scope instead, past the L2, all 256 compute units pull the same few lines from memory: that was
// measured at 5 GB/s a compute unit and set the time of every phase.)
__device__ __forceinline__ int4v load_shared16(const void* p) { return *(GLOBAL_PTR(const int4v))p; }
__device__ __forceinline__ void store_shared8(void* p, unsigned long long v) {
  __hip_atomic_store((GLOBAL_PTR(unsigned long long))p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared4(void* p, unsigned v) {
  __hip_atomic_store((GLOBAL_PTR(unsigned))p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared2(void* p, unsigned short v) {
  __hip_atomic_store((GLOBAL_PTR(unsigned short))p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long pack_bf16x4(const float* v) {
  bf16x4 packed = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
  return __builtin_bit_cast(unsigned long long, packed);
}
__device__ __forceinline__ void store_shared_f32x4(float* p, const float* v) {
  store_shared8(p, (unsigned long long)__float_as_uint(v[0]) | ((unsigned long long)__float_as_uint(v[1]) << 32));
  store_shared8(p + 2, (unsigned long long)__float_as_uint(v[2]) | ((unsigned long long)__float_as_uint(v[3]) << 32));
}

// The same number, but new to the compiler: what is computed from it is computed here and now.
// Every phase of every layer derives the same few dozen offsets from the lane's number; computed
// once and kept (which is what the compiler does when it sees that they are the same), they occupy
// registers that the weights in flight need, and are spilled and reloaded around every use.
__device__ __forceinline__ int fresh(int v) {
  int zero;
  asm volatile("s_mov_b32 %0, 0" : "=s"(zero));
  return v + zero;
}

// A barrier of the work-group that waits for LDS only: loads from memory that are in flight (the
// weights of a later phase) stay in flight.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// The barrier across the grid.  `ahead` issues loads that do not depend on the other work-groups;
// the polling wave issues them only after the barrier has opened, because a wave's loads return
// in order and its polls would queue behind them.
template <typename Ahead>
__device__ __forceinline__ void grid_barrier(unsigned* sync, unsigned epoch, int wave, bool& dead, Ahead&& ahead) {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // this wave's stores are acknowledged
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (wave != 0) {
    ahead();
  } else {
    if (threadIdx.x == 0 && !dead) {
      const unsigned groups = gridDim.x < 8 ? gridDim.x : 8;
      const unsigned g = blockIdx.x & 7, members = (gridDim.x - g + 7) / 8;
      unsigned before = __hip_atomic_fetch_add(&sync[32 + 32 * g], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (before + 1 == epoch * members)
        __hip_atomic_fetch_add(&sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      int spins = 0;
      while (__hip_atomic_load(&sync[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < epoch * groups) {
        ++spins;
        if ((spins & 255) == 0 &&
            __hip_atomic_load(&sync[STACK_SYNC_FAILED], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
          dead = true;
          break;
        }
        if (spins > STACK_SPIN_LIMIT) {
          __hip_atomic_store(&sync[STACK_SYNC_FAILED], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          dead = true;
          break;
        }
      }
    }
    ahead();
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// --- the products ---------------------------------------------------------------------------------
// The weights of U chunks of 32 K values (chunk wave + 8 (u0 + u)) of NT blocks of 16 columns.
template <int NT, int U>
struct Weights {
  int4v w[U][NT];
};

// Which columns of a product with N columns this work-group owns: `cols` of them from n_base, in the
// order of the work-groups or, `reversed`, from the last work-group down, so that the products with
// few columns keep other compute units busy than the remainder of the wide ones.
struct Columns {
  int n_base, n_end, cols, group;
  __device__ __forceinline__ bool any() const { return n_base < n_end; }
};
__device__ __forceinline__ Columns columns_of(int N, int cols, bool reversed) {
  const int slot = reversed ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;
  Columns c;
  c.cols = cols;
  c.group = slot;
  c.n_base = slot * cols;
  c.n_end = c.n_base + cols < N ? c.n_base + cols : N;
  if (c.n_base >= N) c.n_base = c.n_end = N;
  return c;
}

// No load below stands behind a branch of its own: a chunk beyond K, a column beyond the group's
// and a block of columns the group does not have all repeat bytes that are loaded anyway, and
// their products are left out (a scalar branch around the MFMA) or dropped by the epilogue.  With
// a branch per load the compiler keeps a copy of the whole register array for every path.
template <int NT, int U>
__device__ __forceinline__ void issue_weights(Weights<NT, U>& r, GLOBAL_PTR(const bf16_t) packed, int K, Columns cols,
                                              int u0, int wave, int lane_) {
  if (!cols.any()) {                // one branch for the whole set; `multiply` skips this work-group too
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) r.w[u][nt] = int4v{0, 0, 0, 0};
    return;
  }
  const int lane = fresh(lane_);
  const int i16 = lane & 15, g = lane >> 4;
  const int chunks = (K + 31) >> 5;
  // this work-group's block of the packed matrix
  GLOBAL_PTR(const char) block = (GLOBAL_PTR(const char))packed + (int64_t)cols.group * chunks * cols.cols * 64;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int c = wave + STACK_WAVES * (u0 + u);
    c = c < chunks ? c : chunks - 1;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      int j = nt * 16 + i16;
      j = j < cols.cols ? j : cols.cols - 1;
      r.w[u][nt] = *(GLOBAL_PTR(const int4v))(block + (unsigned)((c * cols.cols + j) * 64 + g * 16));
    }
  }
}

// acc += W . A^T over chunks u0 .. u0 + U of this wave; the activations come from `operand(kc)`,
// a lane's eight K values of its row.  BATCH operands are asked for before the first is used.
template <int NT, int U, int BATCH, typename Operand>
__device__ __forceinline__ void multiply(floatx4 (&acc)[NT], const Weights<NT, U>& r, int K, Columns cols, int u0,
                                         int wave, int lane_, Operand&& operand) {
  if (!cols.any()) return;
  const int g = fresh(lane_) >> 4;
  const int chunks = (K + 31) >> 5;
#pragma unroll
  for (int b0 = 0; b0 < U; b0 += BATCH) {
    int4v a[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      if (b0 + j < U) {
        int c = wave + STACK_WAVES * (u0 + b0 + j);
        c = c < chunks ? c : chunks - 1;
        const int k = c * 32 + g * 8;
        a[j] = operand(k < K ? k : K - 8);
      }
    }
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      if (b0 + j < U) {
        if (wave + STACK_WAVES * (u0 + b0 + j) < chunks) {      // (beyond K inside a chunk the packed weights are zero)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, r.w[b0 + j][nt]),
                                                              __builtin_bit_cast(bf16x8, a[j]), acc[nt], 0, 0, 0);
        }
      }
    }
  }
}

// The waves' partial sums meet in LDS; wave nt < NT gets block nt: its lane holds row lane % 16,
// columns 4 (lane / 16) .. + 3 of the block.  Returns whether this wave holds a block.
template <int NT>
__device__ __forceinline__ bool meet(const floatx4 (&acc)[NT], float* red, int wave, int lane_, float (&v)[4]) {
  const int lane = fresh(lane_);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    *reinterpret_cast<floatx4*>(red + ((wave * 2 + nt) * 64 + lane) * 4) = acc[nt];
  lds_barrier();
  if (wave >= NT) return false;
#pragma unroll
  for (int r = 0; r < 4; ++r) v[r] = 0.f;
#pragma unroll
  for (int w = 0; w < STACK_WAVES; ++w) {
    floatx4 part = *reinterpret_cast<const floatx4*>(red + ((w * 2 + wave) * 64 + lane) * 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] += part[r];
  }
  return true;
}

// Normalises the step's rows of the residual stream (read at device scope) into LDS as bfloat16:
// normed[row][width * 2 + 16 bytes].  Wave w takes rows w and w + 8.  QPL quads of floats per lane.
template <int QPL>
__device__ __forceinline__ void normalise_rows(const StackArgs& a, const float* x, int64_t ldx,
                                               GLOBAL_PTR(const float) scale, GLOBAL_PTR(const float) shift, float eps,
                                               unsigned char* normed, int wave, int lane_) {
  const int lane = fresh(lane_);
  const int K = a.width, quads = K >> 2, pitch = K * 2 + 16;
  for (int row = wave; row < a.rows; row += STACK_WAVES) {
    float4 xv[QPL];
    const float* xr = x + (int64_t)row * ldx;
#pragma unroll
    for (int q = 0; q < QPL; ++q) {
      int c = lane + 64 * q;
      int cc = c < quads ? c : 0;
      int4v raw = load_shared16(xr + 4 * cc);
      xv[q] = make_float4(__int_as_float(raw[0]), __int_as_float(raw[1]), __int_as_float(raw[2]), __int_as_float(raw[3]));
    }
    float part = 0.f;
#pragma unroll
    for (int q = 0; q < QPL; ++q)
      if (lane + 64 * q < quads)
        part += a.norm_kind == 0 ? (xv[q].x + xv[q].y + xv[q].z + xv[q].w)
                                 : (xv[q].x * xv[q].x + xv[q].y * xv[q].y + xv[q].z * xv[q].z + xv[q].w * xv[q].w);
    float total = wave_sum(part);
    float mean = 0.f, rstd;
    if (a.norm_kind == 0) {
      mean = total / (float)K;
      float sq = 0.f;
#pragma unroll
      for (int q = 0; q < QPL; ++q)
        if (lane + 64 * q < quads) {
          float a0 = xv[q].x - mean, a1 = xv[q].y - mean, a2 = xv[q].z - mean, a3 = xv[q].w - mean;
          sq += a0 * a0 + a1 * a1 + a2 * a2 + a3 * a3;
        }
      rstd = 1.0f / sqrtf(wave_sum(sq) / (float)K + eps);
    } else {
      rstd = 1.0f / sqrtf(total / (float)K + eps);
    }
#pragma unroll
    for (int q = 0; q < QPL; ++q) {
      int c = lane + 64 * q;
      // (scale and shift are read here, not with the row: fourteen more quads in registers per
      // lane are what the weights in flight need; a lane beyond the row reads its start)
      const float4 gq = load_global_f32x4(scale + 4 * (c < quads ? c : 0));
      const float4 bq = load_global_f32x4((shift ? shift : scale) + 4 * (c < quads ? c : 0));
      if (c < quads) {
        const float on = shift ? 1.f : 0.f;
        bf16x4 y = {(bf16_t)((xv[q].x - mean) * rstd * gq.x + on * bq.x), (bf16_t)((xv[q].y - mean) * rstd * gq.y + on * bq.y),
                    (bf16_t)((xv[q].z - mean) * rstd * gq.z + on * bq.z), (bf16_t)((xv[q].w - mean) * rstd * gq.w + on * bq.w)};
        *reinterpret_cast<bf16x4*>(normed + row * pitch + c * 8) = y;
      }
    }
  }
}

// Attention of the step's one token per sequence: this work-group takes pairs (sequence, key/value
// head) in turn; the eight waves split the keys of a pair and meet in LDS.
__device__ __forceinline__ void attend_pairs(const StackArgs& a, const StackLayer& L, const bf16_t* q_rows, bf16_t* mixed_rows,
                                             float* sm, int wave, int lane_) {
  const int lane = fresh(lane_);
  const int i16 = lane & 15, g = lane >> 4;
  const int group = a.heads / a.kv_heads;
  float* sm_m = sm;                                  // [waves][group]
  float* sm_l = sm + STACK_WAVES * group;            // [waves][group]
  float* sm_o = sm + 2 * STACK_WAVES * group;        // [waves][group][HD]
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bool has_query = i16 < group;
  const int stride = 32 * STACK_WAVES;
  const int ldq = a.heads * HD;
  const float c = L.scale * LOG2_E;
  const int pairs = a.rows * a.kv_heads;
  for (int pair = blockIdx.x; pair < pairs; pair += gridDim.x) {
    const int seq = pair / a.kv_heads, kv_head = pair % a.kv_heads;
    const int head = kv_head * group + (has_query ? i16 : 0);
    const int* block_row = a.blocks + (int64_t)seq * a.max_blocks;
    const int pos = a.positions[seq];
    bf16x8 q[1][NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      int channel = ks * 32 + g * 8;
      q[0][ks] = (has_query && channel < HD)
                     ? __builtin_bit_cast(bf16x8, load_shared16(q_rows + (int64_t)seq * ldq + head * HD + channel))
                     : zero8;
    }
    int qpos[1] = {has_query ? pos : -1};
    floatx4 o[1][ND];
    float m[1] = {-INFINITY}, l[1] = {0.f};
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[0][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    int lo = 0;
    if (a.window > 0 && pos - a.window + 1 > 0) lo = (pos - a.window + 1) & ~31;
    const int first = lo + 32 * wave, end = (pos & ~31) + 32;
    auto fetch = [&](TileOperands& into, int kb) {
      if (kb < end) {
        int block = block_row[kb / BT_KV_BLOCK];
        int64_t plane = ((int64_t)block * a.kv_heads + kv_head) * (int64_t)(BT_KV_BLOCK * HD);
        load_tile(into, (const bf16_t*)(L.keys + plane), (const bf16_t*)(L.values + plane), kb);
      }
    };
    TileOperands current, next;
    fetch(next, first);
    for (int kb = first; kb < end; kb += stride) {
      current = next;
      fetch(next, kb + stride);
      attend_tile<1, true>(current, kb, pos + 1, qpos, a.window, c, q, o, m, l);
    }
    float total = l[0];
    total += __shfl_xor(total, 16, 64);
    total += __shfl_xor(total, 32, 64);
    if (has_query) {
      if (g == 0) {
        sm_m[wave * group + i16] = m[0];
        sm_l[wave * group + i16] = total;
      }
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) sm_o[(wave * group + i16) * HD + dt * 16 + 4 * g + r] = o[0][dt][r];
    }
    lds_barrier();
    for (int e = threadIdx.x; e < group * HD / 2; e += STACK_THREADS) {
      const int j = (2 * e) / HD, channel = (2 * e) % HD;
      float top = sm_m[j];
#pragma unroll
      for (int w = 1; w < STACK_WAVES; ++w) top = fmaxf(top, sm_m[w * group + j]);
      float num0 = 0.f, num1 = 0.f, den = 0.f;
      if (top != -INFINITY) {
#pragma unroll
        for (int w = 0; w < STACK_WAVES; ++w) {
          float f = exp2f(sm_m[w * group + j] - top);
          num0 += sm_o[(w * group + j) * HD + channel] * f;
          num1 += sm_o[(w * group + j) * HD + channel + 1] * f;
          den += sm_l[w * group + j] * f;
        }
      }
      bf16_t r0 = (bf16_t)(den > 0.f ? num0 / den : 0.f), r1 = (bf16_t)(den > 0.f ? num1 / den : 0.f);
      unsigned bits = (unsigned)__builtin_bit_cast(unsigned short, r0) | ((unsigned)__builtin_bit_cast(unsigned short, r1) << 16);
      store_shared4(mixed_rows + (int64_t)seq * ldq + (kv_head * group + j) * HD + channel, bits);
    }
    lds_barrier();     // the next pair writes the same LDS
  }
}

// UW: chunks a wave takes of a product over the width (K <= 256 UW); UD1 + UD2: of the one over the
// inner width; QPL: quads of a row per lane in the norms (width <= 256 QPL).
template <int UW, int UD1, int UD2, int QPL>
__global__ void __launch_bounds__(STACK_THREADS)
decode_stack_kernel(StackArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  // LDS: the waves' partial sums [8][2][64][4] floats, then the normalised rows / attention's scratch
  float* red = reinterpret_cast<float*>(lds);
  unsigned char* normed = lds + STACK_WAVES * 2 * 64 * 4 * sizeof(float);
  const int normed_pitch = a.width * 2 + 16;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int n_q = a.heads * HD, n_kv = a.kv_heads * HD, n_qkv = n_q + 2 * n_kv;
  const Columns cols_qkv = columns_of(n_qkv, a.cols_qkv, false);
  const Columns cols_up = columns_of(a.inner, a.cols_up, false);
  const Columns cols_x = columns_of(a.width, a.cols_x, true);
  const int row = i16 < a.rows ? i16 : a.rows - 1;      // rows beyond the step repeat the last one
  const bool row_real = i16 < a.rows;
  // this lane's part of the residual stream (wave 0 finishes both products that add to it)
  const int x_n0 = cols_x.n_base + 4 * g;
  const bool x_mine = wave == 0 && row_real && x_n0 < cols_x.n_end;
  float x_own[4] = {0.f, 0.f, 0.f, 0.f};
  if (x_mine) {
    float4 v = *reinterpret_cast<const float4*>(a.x + (int64_t)row * a.ldx + x_n0);
    x_own[0] = v.x, x_own[1] = v.y, x_own[2] = v.z, x_own[3] = v.w;
  }
  // where this lane's row keeps its new key and value
  const int my_pos = a.positions[row];
  const int my_block = a.blocks[(int64_t)row * a.max_blocks + my_pos / BT_KV_BLOCK];

  Weights<2, UW> w_qkv;             // (the one set that is asked for in one layer and used in the next)
  unsigned epoch = 0;
  bool dead = false;
  auto tick = [&](int layer, int point) {
    if (a.clocks != nullptr && layer < STACK_CLOCK_LAYERS && threadIdx.x == 0)
      a.clocks[((int64_t)blockIdx.x * STACK_CLOCK_LAYERS + layer) * 10 + point] = wall_clock64();
  };
  issue_weights(w_qkv, a.layers[0].qkv_weight, a.width, cols_qkv, 0, wave, lane);

  const int lane_outside = lane;
  for (int layer = 0; layer < a.n_layers; ++layer) {
    const StackLayer L = a.layers[layer];
    Weights<1, UW> w_out;
    Weights<2, UW> w_up;
    Weights<1, UD1> w_down1;
    Weights<1, UD2> w_down2;
    const int lane = fresh(lane_outside);
    const int i16 = lane & 15, g = lane >> 4;
    const int row = i16 < a.rows ? i16 : a.rows - 1;
    // (each place starts on a cache line of its own: a line that also held bytes written in a later
    // phase would be read, and kept by the reader's L2, before those bytes exist)
    bf16_t* q_rows = a.q + (int64_t)layer * stack_place(a.rows * n_q, 2);
    bf16_t* mixed_rows = a.mixed + (int64_t)layer * stack_place(a.rows * n_q, 2);
    bf16_t* hidden_rows = a.hidden + (int64_t)layer * stack_place(a.rows * a.inner, 2);
    const int64_t between_place = stack_place(a.rows * a.width, 4);
    float* after_mixer = a.between + (int64_t)(2 * layer) * between_place;
    const bool last = layer + 1 == a.n_layers;
    float* after_ff = last ? a.x : after_mixer + between_place;      // the last layer leaves the stream itself
    const int64_t after_ff_pitch = last ? a.ldx : a.width;
    const float* before = layer == 0 ? a.x : after_mixer - between_place;
    const int64_t before_pitch = layer == 0 ? a.ldx : a.width;
    auto ask_out = [&] { issue_weights(w_out, L.out_weight, n_q, cols_x, 0, wave, lane); };
    if (layer == 0) ask_out();
    else grid_barrier(a.sync, ++epoch, wave, dead, ask_out);

    // --- norm, fused projection: queries to the exchange buffer, keys and values to the cache ---
    tick(layer, 0);
    {
      normalise_rows<QPL>(a, before, before_pitch, L.norm1_scale, L.norm1_shift, L.eps1, normed, wave, lane);
      lds_barrier();
      floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
      multiply<2, UW, UW>(acc, w_qkv, a.width, cols_qkv, 0, wave, lane, [&](int kc) {
        return *reinterpret_cast<const int4v*>(normed + row * normed_pitch + kc * 2);
      });
      float v[4];
      if (meet<2>(acc, red, wave, lane, v)) {
        const int n0 = cols_qkv.n_base + wave * 16 + 4 * g;
        if (row_real && n0 < cols_qkv.n_end) {
          if (L.qkv_bias) {
            float4 b = load_global_f32x4(L.qkv_bias + n0);
            v[0] += b.x, v[1] += b.y, v[2] += b.z, v[3] += b.w;
          }
          if (n0 < n_q) {
            store_shared8(q_rows + (int64_t)row * n_q + n0, pack_bf16x4(v));
          } else {
            int c = n0 - n_q;
            const bool is_value = c >= n_kv;
            if (is_value) c -= n_kv;
            const int head = c / HD, channel = c % HD;
            const int64_t base = ((int64_t)my_block * a.kv_heads + head) * (int64_t)(BT_KV_BLOCK * HD);
            if (!is_value) {
              store_shared8((void*)(L.keys + base + key_offset(HD, my_pos, channel)), pack_bf16x4(v));
            } else {
              GLOBAL_PTR(bf16_t) dst = L.values + base + value_offset(HD, my_pos, channel);
#pragma unroll
              for (int i = 0; i < 4; ++i) store_shared2((void*)(dst + 4 * i), __builtin_bit_cast(unsigned short, (bf16_t)v[i]));
            }
          }
        }
      }
    }
    tick(layer, 1);
    grid_barrier(a.sync, ++epoch, wave, dead, [] {});

    // --- attention ---
    tick(layer, 2);
    attend_pairs(a, L, q_rows, mixed_rows, reinterpret_cast<float*>(normed), wave, lane);
    tick(layer, 3);
    grid_barrier(a.sync, ++epoch, wave, dead, [&] { issue_weights(w_up, L.up_weight, a.width, cols_up, 0, wave, lane); });

    // --- output projection into the residual stream ---
    tick(layer, 4);
    {
      floatx4 acc[1] = {floatx4{0.f, 0.f, 0.f, 0.f}};
      multiply<1, UW, UW>(acc, w_out, n_q, cols_x, 0, wave, lane,
                          [&](int kc) { return load_shared16(mixed_rows + (int64_t)row * n_q + kc); });
      float v[4];
      if (meet<1>(acc, red, wave, lane, v) && x_mine) {
        if (L.out_bias) {
          float4 b = load_global_f32x4(L.out_bias + x_n0);
          v[0] += b.x, v[1] += b.y, v[2] += b.z, v[3] += b.w;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) x_own[i] += v[i];
        store_shared_f32x4(after_mixer + (int64_t)row * a.width + x_n0, x_own);
      }
    }
    tick(layer, 5);
    grid_barrier(a.sync, ++epoch, wave, dead,
                 [&] { issue_weights(w_down1, L.down_weight, a.inner, cols_x, 0, wave, lane); });

    // --- norm, feed-forward in, activation ---
    tick(layer, 6);
    {
      normalise_rows<QPL>(a, after_mixer, a.width, L.norm2_scale, L.norm2_shift, L.eps2, normed, wave, lane);
      lds_barrier();
      floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
      multiply<2, UW, UW>(acc, w_up, a.width, cols_up, 0, wave, lane, [&](int kc) {
        return *reinterpret_cast<const int4v*>(normed + row * normed_pitch + kc * 2);
      });
      issue_weights(w_down2, L.down_weight, a.inner, cols_x, UD1, wave, lane);
      float v[4];
      if (meet<2>(acc, red, wave, lane, v)) {
        const int n0 = cols_up.n_base + wave * 16 + 4 * g;
        if (row_real && n0 < cols_up.n_end) {
          if (L.up_bias) {
            float4 b = load_global_f32x4(L.up_bias + n0);
            v[0] += b.x, v[1] += b.y, v[2] += b.z, v[3] += b.w;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = activate<bf16_t>(v[i], a.act);
          store_shared8(hidden_rows + (int64_t)row * a.inner + n0, pack_bf16x4(v));
        }
      }
    }
    tick(layer, 7);
    grid_barrier(a.sync, ++epoch, wave, dead, [] {});

    // --- feed-forward out into the residual stream ---
    tick(layer, 8);
    {
      floatx4 acc[1] = {floatx4{0.f, 0.f, 0.f, 0.f}};
      auto operand = [&](int kc) { return load_shared16(hidden_rows + (int64_t)row * a.inner + kc); };
      multiply<1, UD1, 7>(acc, w_down1, a.inner, cols_x, 0, wave, lane, operand);
      multiply<1, UD2, 6>(acc, w_down2, a.inner, cols_x, UD1, wave, lane, operand);
      // (unconditionally: behind a branch the old set would have to stay alive through the whole
      // layer beside the new one; the last layer asks for its own weights again and drops them)
      issue_weights(w_qkv, a.layers[layer + 1 < a.n_layers ? layer + 1 : layer].qkv_weight, a.width, cols_qkv, 0, wave, lane);
      float v[4];
      if (meet<1>(acc, red, wave, lane, v) && x_mine) {
        if (L.down_bias) {
          float4 b = load_global_f32x4(L.down_bias + x_n0);
          v[0] += b.x, v[1] += b.y, v[2] += b.z, v[3] += b.w;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) x_own[i] += v[i];
        store_shared_f32x4(after_ff + (int64_t)row * after_ff_pitch + x_n0, x_own);
      }
    }
    tick(layer, 9);
  }
}

// What the kernel takes; a stack outside it runs layer by layer through the separate kernels.
BT_EXPORT int bt_decode_stack(void* stream, const StackArgs* args, int grid) {
  const StackArgs& a = *args;
  constexpr int UW = 7, UD1 = 13, UD2 = 12, QPL = 7;
  if (a.n_layers <= 0 || a.rows <= 0) return BT_OK;
  if (a.rows > STACK_MAX_ROWS) BT_REFUSE("decode_stack: %d rows, at most %d", a.rows, STACK_MAX_ROWS);
  if (grid < 1 || grid > 1024) BT_REFUSE("decode_stack: a grid of %d work-groups", grid);
  if (a.heads <= 0 || a.kv_heads <= 0 || a.heads % a.kv_heads != 0 || a.heads / a.kv_heads > 16)
    BT_REFUSE("decode_stack: %d query heads over %d key/value heads (at most 16 share one)", a.heads, a.kv_heads);
  if (a.width % 8 != 0 || a.width > 256 * UW || a.width > 256 * QPL || a.ldx % 4 != 0)
    BT_REFUSE("decode_stack: width %d must be a multiple of 8 up to %d", a.width, 256 * (UW < QPL ? UW : QPL));
  if (a.heads * HD > 256 * UW) BT_REFUSE("decode_stack: %d heads of %d, at most %d channels", a.heads, HD, 256 * UW);
  if (a.inner % 8 != 0 || a.inner > 256 * (UD1 + UD2))
    BT_REFUSE("decode_stack: inner width %d must be a multiple of 8 up to %d", a.inner, 256 * (UD1 + UD2));
  const int n_qkv = (a.heads + 2 * a.kv_heads) * HD;
  if (a.cols_qkv < 4 || a.cols_qkv > 32 || a.cols_qkv % 4 || a.cols_up < 4 || a.cols_up > 32 || a.cols_up % 4 ||
      a.cols_x < 4 || a.cols_x > 16 || a.cols_x % 4)
    BT_REFUSE("decode_stack: columns per work-group %d, %d, %d must be multiples of four up to 32, 32, 16",
              a.cols_qkv, a.cols_up, a.cols_x);
  if ((int64_t)grid * a.cols_qkv < n_qkv || (int64_t)grid * a.cols_up < a.inner || (int64_t)grid * a.cols_x < a.width)
    BT_REFUSE("decode_stack: %d work-groups cannot hold %d, %d and %d columns", grid, n_qkv, a.inner, a.width);
  if (a.norm_kind != 0 && a.norm_kind != 1) BT_REFUSE("decode_stack: unknown norm %d", a.norm_kind);
  if (a.act != ACT_GELU_TANH && a.act != ACT_GELU_ERF) BT_REFUSE("decode_stack: unknown activation %d", a.act);
  if (((uintptr_t)a.q | (uintptr_t)a.mixed | (uintptr_t)a.hidden | (uintptr_t)a.between) & 255)
    BT_REFUSE("decode_stack: the exchange buffers must be 256-byte aligned");
  if (!a.layers || !a.x || !a.blocks || !a.positions || !a.q || !a.mixed || !a.hidden || !a.between || !a.sync)
    BT_REFUSE("decode_stack: a null argument");
  const int group = a.heads / a.kv_heads;
  size_t work = (size_t)STACK_MAX_ROWS * (a.width * 2 + 16);
  size_t attn = (size_t)(2 * STACK_WAVES * group + STACK_WAVES * group * HD) * sizeof(float);
  size_t lds = (size_t)STACK_WAVES * 2 * 64 * 4 * sizeof(float) + (work > attn ? work : attn);
  if (lds > 160 * 1024) BT_REFUSE("decode_stack: %zu bytes of LDS, at most 160 KB", lds);
  auto kernel = decode_stack_kernel<UW, UD1, UD2, QPL>;
  static size_t granted = 0;
  if (lds > granted) {
    hipError_t err = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) BT_REFUSE("decode_stack: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
    granted = lds;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(STACK_THREADS), lds, (hipStream_t)stream, a);
  return bt_check_launch("decode_stack");
}

BT_EXPORT long long bt_decode_stack_place(long long elements, int element_bytes) {
  return stack_place(elements, element_bytes);
}
BT_EXPORT int bt_decode_stack_sync_words() { return STACK_SYNC_WORDS; }
BT_EXPORT int bt_decode_stack_failed_word() { return STACK_SYNC_FAILED; }
BT_EXPORT int bt_decode_stack_clock_layers() { return STACK_CLOCK_LAYERS; }
