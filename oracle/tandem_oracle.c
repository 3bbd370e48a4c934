/* CPU oracle for tandem's data-parallel reduction path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain C restatement of the arithmetic of the reference's Python engine, used
 * by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as
 * the checker. The library under tandem_amd/ never links, loads or calls it.
 *
 * What each function follows in the reference:
 *   orc_ring_fold_*      tandem/comm.py:336-343 (divide the whole tensor first),
 *                        comm.py:301-305 (ring reduce-scatter step order),
 *                        comm.py:275-277 (into.add_(slot): into + slot).
 *   orc_ring_partial_*   the same recurrence stopped early: what a non-owner
 *                        rank holds after a bare reduce_scatter (comm.py:350-352).
 *   orc_adamw_*          tandem/optim.py:16-37, with the operation order of
 *                        torch's single-tensor AdamW on CPU (lerp_ and addcmul_
 *                        fuse their last multiply-add, addcdiv_ does not).
 *
 * What pins them (tests/test_oracle_ring.py, test_oracle_adamw.py, test_oracle_cpu_engine.py): outputs of the
 * reference's own engine and optimizer kept as fixtures in tests/golden (ring_w2/3/4.npz and ring_dtypes_w3.npz:
 * whole buffers, partial sums included; adamw.npz; adamw_dtypes.npz for float64, bfloat16 and float16 shards), a
 * message-by-message simulator of the ring written independently of the closed form, torch's single-tensor AdamW,
 * float64 recurrences and all 65,536 half-precision bit patterns. No function here is without such a check.
 *
 * Built with -ffp-contract=off: every fused multiply-add below is explicit.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- 16-bit floats as bit patterns: widen exactly, round to nearest even once.
 * A NaN narrows to the canonical quiet NaN of the type (bf16 0x7fc0, f16 0x7e00): sign and payload of a
 * NaN are not kept. torch's own conversions do not agree on them from build to build (this container's CPU
 * build narrows a float NaN to bf16 0xffff), so the reference's outputs pin no NaN bits, only where the NaNs are. */
static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)0x7fc0u; /* the canonical quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

static float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)0x7e00u; /* the canonical quiet NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536: inf (65520 rounds up too, below) */
  if (a >= 0x38800000u) {                                  /* normal half */
    uint32_t m = a - 0x38000000u;                          /* rebias */
    uint32_t lsb = (m >> 13) & 1u;
    m += 0x0fffu + lsb;
    return (uint16_t)(sign | (m >> 13)); /* a carry into the exponent is the right answer, up to inf */
  }
  if (a < 0x33000000u) return (uint16_t)sign; /* < 2^-25: rounds to zero */
  /* subnormal half: value = man24 * 2^(e-150); target unit 2^-24 */
  uint32_t e = a >> 23;
  uint32_t man = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift = 126u - e; /* 14..24 */
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | q);
}

/* ---- ring fold: the value of chunk `c` after the ring reduce-scatter.
 *
 * y_q = x_q / n (true division, whole tensor first, only for "avg"), then
 *   acc = y[(c+1) % n];  for k = 2..n: acc = y[(c+k) % n] + acc
 * so rank c's own term is added last. `upto` stops the recurrence after rank
 * (c+upto) % n has added its term (upto = n: the full sum; upto = 1: the bare,
 * divided input of rank c+1), which is what rank (c+upto) % n holds in chunk c
 * after a bare reduce_scatter. */
#define RING_FOLD(NAME, T, ACC, LOAD, STORE, DIVTYPE)                                                        \
  void NAME(const T* const* x, int n, int c, int upto, int average, int64_t lo, int64_t hi, T* out) {       \
    const DIVTYPE d = (DIVTYPE)n;                                                                            \
    for (int64_t i = lo; i < hi; ++i) {                                                                      \
      ACC acc = LOAD(x[(c + 1) % n][i]);                                                                     \
      if (average) acc = LOAD(STORE((ACC)(acc / d)));                                                        \
      for (int k = 2; k <= upto; ++k) {                                                                      \
        ACC y = LOAD(x[(c + k) % n][i]);                                                                     \
        if (average) y = LOAD(STORE((ACC)(y / d)));                                                          \
        acc = LOAD(STORE((ACC)(y + acc)));                                                                   \
      }                                                                                                      \
      out[i - lo] = STORE(acc);                                                                              \
    }                                                                                                        \
  }

#define IDENT(v) (v)
RING_FOLD(orc_ring_fold_f32, float, float, IDENT, IDENT, float)
RING_FOLD(orc_ring_fold_f64, double, double, IDENT, IDENT, double)
RING_FOLD(orc_ring_fold_bf16, uint16_t, float, bf16_to_f32, f32_to_bf16, float)
RING_FOLD(orc_ring_fold_f16, uint16_t, float, f16_to_f32, f32_to_f16, float)
RING_FOLD(orc_ring_fold_i64, int64_t, int64_t, IDENT, IDENT, int64_t)
/* The narrower integers: ATen's add_ wraps around (the reference adds whatever dtype it is given with
 * into.add_(slot), tandem/comm.py:276-277), so the sums are taken in unsigned arithmetic of the element's
 * own width, which is the two's-complement sum of signed elements bit for bit. Never averaged. */
#define TO_U16(v) ((uint16_t)(v))
#define TO_U8(v) ((uint8_t)(v))
RING_FOLD(orc_ring_fold_u32, uint32_t, uint32_t, IDENT, IDENT, uint32_t)
RING_FOLD(orc_ring_fold_u16, uint16_t, uint32_t, IDENT, TO_U16, uint32_t)
RING_FOLD(orc_ring_fold_u8, uint8_t, uint32_t, IDENT, TO_U8, uint32_t)

/* Conversions exported so tests can check them against numpy / torch. */
void orc_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_f32(in[i]);
}
void orc_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16(in[i]);
}
void orc_f16_to_f32(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f16_to_f32(in[i]);
}
void orc_f32_to_f16(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f32_to_f16(in[i]);
}

/* ---- AdamW, one step over one shard (tandem/optim.py:16-37).
 *
 * The scalars arrive already rounded the way torch applies a Python double to a
 * float tensor (rounded to fp32 once):
 *   decay     = f32(1 - lr*wd)          optim.py:28-29   (use_decay = wd != 0)
 *   w1        = f32(1 - beta1)          optim.py:30      lerp_ weight
 *   beta2     = f32(beta2)              optim.py:31
 *   one_m_b2  = f32(1 - beta2)          optim.py:31      addcmul_ value
 *   bc2_sqrt  = f32((1 - beta2**t)**.5) optim.py:33-36
 *   eps       = f32(eps)                optim.py:36
 *   neg_step  = f32(-(lr / (1 - beta1**t)))   optim.py:32-34,37
 *
 * Phase A: decay, first and second moment.  Phase B: the parameter update from
 * a given sqrt(v).  orc_adamw_f32 runs both with the correctly rounded sqrtf. */
void orc_adamw_moments_f32(float* p, const float* g, float* m, float* v, int64_t n, int use_decay, float decay,
                           float w1, float beta2, float one_m_b2) {
  for (int64_t i = 0; i < n; ++i) {
    if (use_decay) p[i] = p[i] * decay;
    const float diff = g[i] - m[i];
    /* lerp_: weight < 0.5 ? fma(w, end-start, start) : fma(w-1, end-start, end) */
    m[i] = fabsf(w1) < 0.5f ? fmaf(w1, diff, m[i]) : fmaf(w1 - 1.0f, diff, g[i]);
    const float vs = v[i] * beta2;
    v[i] = fmaf(one_m_b2 * g[i], g[i], vs); /* addcmul_: (value*t1) rounded, then fused */
  }
}

void orc_adamw_apply_f32(float* p, const float* m, const float* sqrt_v, int64_t n, float bc2_sqrt, float eps,
                         float neg_step) {
  for (int64_t i = 0; i < n; ++i) {
    const float d = sqrt_v[i] / bc2_sqrt + eps;
    p[i] = p[i] + (neg_step * m[i]) / d; /* addcdiv_: (value*t1)/t2, then add; nothing fused */
  }
}

void orc_adamw_f32(float* p, const float* g, float* m, float* v, int64_t n, int use_decay, float decay, float w1,
                   float beta2, float one_m_b2, float bc2_sqrt, float eps, float neg_step) {
  orc_adamw_moments_f32(p, g, m, v, n, use_decay, decay, w1, beta2, one_m_b2);
  for (int64_t i = 0; i < n; ++i) {
    const float d = sqrtf(v[i]) / bc2_sqrt + eps;
    p[i] = p[i] + (neg_step * m[i]) / d;
  }
}

/* ---- AdamW on float64 shards: the same operations on doubles (tandem/optim.py:28-37 takes any floating dtype).
 * A Python double applied to a double tensor is used as it is, so the scalars arrive unrounded. lerp_ and
 * addcmul_ fuse their last multiply-add on doubles as on floats, tensor / scalar is a true division,
 * addcdiv_ is (value*m)/d then the add: checked operation by operation against torch's CPU kernels. */
void orc_adamw_moments_f64(double* p, const double* g, double* m, double* v, int64_t n, int use_decay, double decay,
                           double w1, double beta2, double one_m_b2) {
  for (int64_t i = 0; i < n; ++i) {
    if (use_decay) p[i] = p[i] * decay;
    const double diff = g[i] - m[i];
    m[i] = fabs(w1) < 0.5 ? fma(w1, diff, m[i]) : fma(w1 - 1.0, diff, g[i]);
    const double vs = v[i] * beta2;
    v[i] = fma(one_m_b2 * g[i], g[i], vs);
  }
}

void orc_adamw_apply_f64(double* p, const double* m, const double* sqrt_v, int64_t n, double bc2_sqrt, double eps,
                         double neg_step) {
  for (int64_t i = 0; i < n; ++i) {
    const double d = sqrt_v[i] / bc2_sqrt + eps;
    p[i] = p[i] + (neg_step * m[i]) / d;
  }
}

void orc_adamw_f64(double* p, const double* g, double* m, double* v, int64_t n, int use_decay, double decay, double w1,
                   double beta2, double one_m_b2, double bc2_sqrt, double eps, double neg_step) {
  orc_adamw_moments_f64(p, g, m, v, n, use_decay, decay, w1, beta2, one_m_b2);
  for (int64_t i = 0; i < n; ++i) {
    const double d = sqrt(v[i]) / bc2_sqrt + eps;
    p[i] = p[i] + (neg_step * m[i]) / d;
  }
}

/* ---- AdamW on bfloat16 and float16 shards (bit patterns). Every one of the torch operations of tandem/optim.py:28-37 reads
 * 16-bit tensors, computes in fp32 (ATen's opmath; the Python scalars rounded to fp32, not to the 16-bit type) and writes a
 * 16-bit tensor, so the result is rounded to nearest even after EACH operation: p*decay; the lerp; v*beta2; the addcmul;
 * the sqrt; the division; + eps; the addcdiv. One scalar is narrower than the others: add_(eps) adds eps ROUNDED TO
 * THE 16-BIT TYPE (float16 turns the usual 1e-8 into 0, and an element whose gradients were all zero into 0/0) (ATen wraps the scalar of an add in the tensor's dtype), where mul_, lerp_, addcmul_, the division and addcdiv_
 * take theirs as fp32 (checked operation by operation against torch's CPU kernels on values where the two differ).
 * Inside an operation the fp32 arithmetic is that of the fp32 kernels
 * above. As for fp32 the step comes in two phases, so that a test can put torch's own bf16 square roots between them. */
/* The three functions for one 16-bit type: NAME = bf16 or f16, W widens its bit pattern to fp32, N narrows (nearest even). */
#define ADAMW_16(NAME, W, N)                                                                                              \
  void orc_adamw_moments_##NAME(uint16_t* p, const uint16_t* g, uint16_t* m, uint16_t* v, int64_t n, int use_decay,       \
                                float decay, float w1, float beta2, float one_m_b2) {                                     \
    for (int64_t i = 0; i < n; ++i) {                                                                                     \
      const float G = W(g[i]);                                                                                            \
      float M = W(m[i]), V = W(v[i]);                                                                                     \
      if (use_decay) p[i] = N(W(p[i]) * decay);                                                                           \
      const float diff = G - M; /* inside lerp_: not rounded to the 16-bit type */                                        \
      m[i] = N(fabsf(w1) < 0.5f ? fmaf(w1, diff, M) : fmaf(w1 - 1.0f, diff, G));                                          \
      V = W(N(V * beta2));                                                                                                \
      v[i] = N(fmaf(one_m_b2 * G, G, V));                                                                                 \
    }                                                                                                                     \
  }                                                                                                                       \
  void orc_adamw_apply_##NAME(uint16_t* p, const uint16_t* m, const uint16_t* sqrt_v, int64_t n, float bc2_sqrt,          \
                              float eps, float neg_step) {                                                                \
    for (int64_t i = 0; i < n; ++i) {                                                                                     \
      float D = W(N(W(sqrt_v[i]) / bc2_sqrt));                                                                            \
      D = W(N(D + W(N(eps))));                                                                                            \
      p[i] = N(W(p[i]) + (neg_step * W(m[i])) / D);                                                                       \
    }                                                                                                                     \
  }                                                                                                                       \
  void orc_adamw_##NAME(uint16_t* p, const uint16_t* g, uint16_t* m, uint16_t* v, int64_t n, int use_decay, float decay,  \
                        float w1, float beta2, float one_m_b2, float bc2_sqrt, float eps, float neg_step) {               \
    orc_adamw_moments_##NAME(p, g, m, v, n, use_decay, decay, w1, beta2, one_m_b2);                                       \
    for (int64_t i = 0; i < n; ++i) {                                                                                     \
      float D = W(N(sqrtf(W(v[i]))));                                                                                     \
      D = W(N(D / bc2_sqrt));                                                                                             \
      D = W(N(D + W(N(eps))));                                                                                            \
      p[i] = N(W(p[i]) + (neg_step * W(m[i])) / D);                                                                       \
    }                                                                                                                     \
  }

ADAMW_16(bf16, bf16_to_f32, f32_to_bf16)
ADAMW_16(f16, f16_to_f32, f32_to_f16)
