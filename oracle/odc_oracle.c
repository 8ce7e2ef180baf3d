/*
 * Scalar C restatement of the arithmetic on ODC's gather / scatter-accumulate path.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libodc_oracle.so and loaded by tests/ to pin the
 * torch-CPU oracle (oracle/odc_oracle.py) with an independent implementation. Nothing in the
 * product links or loads it.
 *
 * Compile with -ffp-contract=off and without -ffast-math so that every add below is exactly
 * one IEEE-754 binary32 addition.
 */
#include <stdint.h>
#include <string.h>

static float widen_bf16(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* IEEE binary16 -> binary32, exact, by field manipulation (no compiler half support needed) */
static float widen_f16(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t narrow_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN */
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16); /* round to nearest even */
}

/* gather, odc/primitives/gather.py:116-127: out.view(W,-1)[r] = shard_r, bytes */
void oracle_gather(uint8_t* out, const uint8_t* const* shards, uint32_t world, uint64_t shard_bytes) {
  for (uint32_t r = 0; r < world; ++r) memcpy(out + (uint64_t)r * shard_bytes, shards[r], shard_bytes);
}

/* scatter-accumulate, odc/primitives/scatter_accumulate.py:386 with buf = chunk r of the
 * gradient (:659-669): acc_r[i] += grad[r*S + i]; elements at index >= grad_elems are +0
 * (odc/fsdp/fsdp1.py:25-38). grad_kind: 0 bf16, 1 fp16, 2 fp32. fp32 accumulation. */
void oracle_scatter_accumulate_f32(float* const* accs, const void* grad, int grad_kind,
                                   uint64_t grad_elems, uint32_t world, uint64_t shard_elems) {
  for (uint32_t r = 0; r < world; ++r) {
    float* acc = accs[r];
    for (uint64_t i = 0; i < shard_elems; ++i) {
      uint64_t gi = (uint64_t)r * shard_elems + i;
      float g = 0.0f;
      if (gi < grad_elems) {
        if (grad_kind == 0) g = widen_bf16(((const uint16_t*)grad)[gi]);
        else if (grad_kind == 1) g = widen_f16(((const uint16_t*)grad)[gi]);
        else g = ((const float*)grad)[gi];
      }
      volatile float s = acc[i] + g;
      acc[i] = s;
    }
  }
}

/* bf16 accumulation of bf16 gradients: widen both, one fp32 add, round to nearest even */
void oracle_scatter_accumulate_bf16(uint16_t* const* accs, const uint16_t* grad, uint64_t grad_elems,
                                    uint32_t world, uint64_t shard_elems) {
  for (uint32_t r = 0; r < world; ++r) {
    uint16_t* acc = accs[r];
    for (uint64_t i = 0; i < shard_elems; ++i) {
      uint64_t gi = (uint64_t)r * shard_elems + i;
      float g = gi < grad_elems ? widen_bf16(grad[gi]) : 0.0f;
      volatile float s = widen_bf16(acc[i]) + g;
      acc[i] = narrow_bf16(s);
    }
  }
}

void oracle_widen_bf16(float* out, const uint16_t* in, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) out[i] = widen_bf16(in[i]);
}

void oracle_widen_f16(float* out, const uint16_t* in, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) out[i] = widen_f16(in[i]);
}

void oracle_narrow_bf16(uint16_t* out, const float* in, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) out[i] = narrow_bf16(in[i]);
}

/* acc[i] /= divisor: one binary32 division, correctly rounded (the divide of
 * odc/fsdp/fsdp2.py:846-847 and of _div_if_needed, odc/fsdp/fsdp1.py:324-330). */
void oracle_divide_f32(float* acc, float divisor, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) {
    volatile float q = acc[i] / divisor;
    acc[i] = q;
  }
}
