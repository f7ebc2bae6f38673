// Synthetic-model weight writer: fills device buffers with random-init weights already quantized to GGUF blocks, so an
// 8B-parameter model can be materialised in HBM in well under a second (the reference has no quantizer: its weights arrive
// quantized inside GGUF files; benchmark configuration 3 asks for random-init weights quantized to Q4_0 with a Q6_K lm-head).
// Values: w = amp * (2u - 1), u = 24-bit uniform from a murmur3-finalizer hash of (seed, element index), i.e. U(-amp, amp)
// like nn.Linear's init U(-1/sqrt(in), 1/sqrt(in)) (tinygrad/nn/__init__.py:173-174).
// Q4_0 uses ggml's reference rule (d = signed max / -8, q = min(15, int(x / d + 8.5))); Q6_K uses a plain absmax rule per
// 16-group (sub-scale = amax / 31 quantized to int8 against d = max sub-scale / 127).  Either way the result is just a valid
// block stream: parity tests read the bytes back and hand the same bytes to the oracle.
#include "common.h"
#include "host.h"

__device__ __forceinline__ uint32_t fmix32(uint32_t h) { h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16; return h; }
__device__ __forceinline__ float rnd_uniform(uint32_t seed, uint64_t idx, float amp) {
  const uint32_t h = fmix32((uint32_t)idx * 0x9E3779B1u + fmix32(seed ^ (uint32_t)(idx >> 32)));
  return amp * ((float)(h >> 8) * (2.0f / 16777216.0f) - 1.0f);
}

__global__ __launch_bounds__(256) void synth_q4_0_kernel(uint8_t* __restrict__ out, int64_t nblocks, uint32_t seed, float amp) {
  for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
    float x[32]; float amax = 0.f, mx = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++) { x[j] = rnd_uniform(seed, (uint64_t)b * 32 + j, amp); if (fabsf(x[j]) > amax) { amax = fabsf(x[j]); mx = x[j]; } }
    const float d = mx / -8.0f, id = d != 0.f ? 1.0f / d : 0.f;
    uint8_t* o = out + b * 18;
    const uint32_t dh = f2h_bits(d);
    o[0] = dh & 0xFF; o[1] = dh >> 8;
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const int q0 = min(15, (int)(x[j] * id + 8.5f)), q1 = min(15, (int)(x[j + 16] * id + 8.5f));
      o[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

// Q8_0: d = amax / 127, q = round(x / d) (ggml's reference rule)
__global__ __launch_bounds__(256) void synth_q8_0_kernel(uint8_t* __restrict__ out, int64_t nblocks, uint32_t seed, float amp) {
  for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
    float x[32]; float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++) { x[j] = rnd_uniform(seed, (uint64_t)b * 32 + j, amp); amax = fmaxf(amax, fabsf(x[j])); }
    const float d = amax / 127.0f, id = d != 0.f ? 1.0f / d : 0.f;
    uint8_t* o = out + b * 34;
    const uint32_t dh = f2h_bits(d);
    o[0] = dh & 0xFF; o[1] = dh >> 8;
#pragma unroll
    for (int j = 0; j < 32; j++) o[2 + j] = (uint8_t)(int8_t)max(-127, min(127, (int)rintf(x[j] * id)));
  }
}

__global__ __launch_bounds__(256) void synth_q6_k_kernel(uint8_t* __restrict__ out, int64_t nblocks, uint32_t seed, float amp) {
  for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
    uint8_t* o = out + b * 210;
    float s[16]; float smax = 0.f;
    for (int g = 0; g < 16; g++) {
      float am = 0.f;
      for (int i = 0; i < 16; i++) am = fmaxf(am, fabsf(rnd_uniform(seed, (uint64_t)b * 256 + g * 16 + i, amp)));
      s[g] = am / 31.0f; smax = fmaxf(smax, s[g]);
    }
    const uint32_t dh = f2h_bits(smax / 127.0f);
    const float d = h2f_bits(dh);
    for (int i = 0; i < 192; i++) o[i] = 0;
    for (int g = 0; g < 16; g++) {
      int sc = d > 0.f ? (int)rintf(s[g] / d) : 0; sc = max(-128, min(127, sc));
      o[192 + g] = (uint8_t)(int8_t)sc;
      const float eff = d * (float)sc;
      for (int i = 0; i < 16; i++) {
        const int e = g * 16 + i;                       // element within the superblock: 128*half + 32*j + l
        const float x = rnd_uniform(seed, (uint64_t)b * 256 + e, amp);
        int q = eff != 0.f ? (int)rintf(x / eff) : 0; q = max(-32, min(31, q));
        const int u = q + 32, half = e >> 7, j = (e >> 5) & 3, l = e & 31;
        uint8_t* ql = o + 64 * half + ((j & 1) ? 32 : 0) + l;
        *ql |= (uint8_t)((u & 0xF) << ((j & 2) ? 4 : 0));
        o[128 + 32 * half + l] |= (uint8_t)((u >> 4) << (2 * j));
      }
    }
    o[208] = dh & 0xFF; o[209] = dh >> 8;
  }
}

__global__ __launch_bounds__(256) void synth_f16_kernel(_Float16* __restrict__ out, int64_t n, uint32_t seed, float amp) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) out[i] = (_Float16)rnd_uniform(seed, (uint64_t)i, amp);
}
// MXFP4 blocks: E2M1 nibbles uniform in 0..15, E8M0 byte uniform in [127 + lo, 127 + hi] (effective block scale 2^lo..2^hi on
// the true E2M1 values; under the reference's decode that is 2^(e-128) times the doubled table: the same number)
__global__ __launch_bounds__(256) void synth_mxfp4_kernel(uint8_t* __restrict__ out, int64_t nblocks, uint32_t seed, int lo, int hi) {
  for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
    uint8_t* o = out + b * 17;
    const uint32_t h = fmix32((uint32_t)b * 0x9E3779B1u + fmix32(seed ^ (uint32_t)(b >> 32) ^ 0x5bd1e995u));
    o[0] = (uint8_t)(127 + lo + (int)(h % (uint32_t)(hi - lo + 1)));
    for (int j = 0; j < 4; j++) {
      const uint32_t r = fmix32(h + 0x9E3779B9u * (j + 1));
      o[1 + 4 * j] = r & 0xFF; o[2 + 4 * j] = (r >> 8) & 0xFF; o[3 + 4 * j] = (r >> 16) & 0xFF; o[4 + 4 * j] = r >> 24;
    }
  }
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ out, int64_t n, float value) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) out[i] = value;
}

// Q4_K: a min/max rule per 32-weight sub-block (min m = max(0, -min x), scale s = (max x + m) / 15), superblock d = max s / 63 and
// dmin = max m / 63 in fp16, 6-bit sc = round(s / d), mn = round(m / dmin), q = clamp(round((x + dmin mn) / (d sc)), 0, 15), packed as
// ggml's block_q4_K (get_scale_min_k4 layout).  Not ggml's iterative search: just a valid block stream of the right magnitude.
__global__ __launch_bounds__(256) void synth_q4_k_kernel(uint8_t* __restrict__ out, int64_t nblocks, uint32_t seed, float amp) {
  for (int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x; b < nblocks; b += (int64_t)gridDim.x * 256) {
    uint8_t* o = out + b * 144;
    float s[8], m[8]; float smax = 0.f, mmax = 0.f;
    for (int g = 0; g < 8; g++) {
      float lo = 0.f, hi = 0.f;
      for (int i = 0; i < 32; i++) { const float x = rnd_uniform(seed, (uint64_t)b * 256 + g * 32 + i, amp); lo = fminf(lo, x); hi = fmaxf(hi, x); }
      m[g] = -lo; s[g] = (hi + m[g]) / 15.0f; smax = fmaxf(smax, s[g]); mmax = fmaxf(mmax, m[g]);
    }
    const uint32_t dh = f2h_bits(smax / 63.0f), mh = f2h_bits(mmax / 63.0f);
    const float d = h2f_bits(dh), dmin = h2f_bits(mh);
    o[0] = dh & 0xFF; o[1] = dh >> 8; o[2] = mh & 0xFF; o[3] = mh >> 8;
    int sc[8], mn[8];
    for (int g = 0; g < 8; g++) { sc[g] = d > 0.f ? min(63, (int)rintf(s[g] / d)) : 0; mn[g] = dmin > 0.f ? min(63, (int)rintf(m[g] / dmin)) : 0; }
    for (int j = 0; j < 4; j++) {
      o[4 + j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
      o[8 + j] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
      o[12 + j] = (uint8_t)((sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4));
    }
    for (int p = 0; p < 4; p++) {                              // qs[32 p + i]: low nibble = sub-block 2p, high nibble = sub-block 2p + 1
      for (int i = 0; i < 32; i++) {
        int q[2];
        for (int h = 0; h < 2; h++) {
          const int g = 2 * p + h;
          const float eff = d * (float)sc[g], x = rnd_uniform(seed, (uint64_t)b * 256 + g * 32 + i, amp);
          q[h] = eff > 0.f ? max(0, min(15, (int)rintf((x + dmin * (float)mn[g]) / eff))) : 0;
        }
        o[16 + 32 * p + i] = (uint8_t)(q[0] | (q[1] << 4));
      }
    }
  }
}

extern "C" int tga_synth_weights(int ggml_type, void* out, int64_t n_elements, uint32_t seed, float amp, void* stream) {
  TGA_REQUIRE(out && n_elements >= 0, "tga_synth_weights: bad argument");
  hipStream_t s = (hipStream_t)stream;
  if (n_elements == 0) return 0;
  if (ggml_type == GGML_Q4_0) {
    TGA_REQUIRE(n_elements % 32 == 0, "tga_synth_weights: Q4_0 needs a multiple of 32 elements");
    const int64_t nb = n_elements / 32; const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
    synth_q4_0_kernel<<<grid, 256, 0, s>>>((uint8_t*)out, nb, seed, amp);
  } else if (ggml_type == GGML_Q8_0) {
    TGA_REQUIRE(n_elements % 32 == 0, "tga_synth_weights: Q8_0 needs a multiple of 32 elements");
    const int64_t nb = n_elements / 32; const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
    synth_q8_0_kernel<<<grid, 256, 0, s>>>((uint8_t*)out, nb, seed, amp);
  } else if (ggml_type == GGML_Q6_K) {
    TGA_REQUIRE(n_elements % 256 == 0, "tga_synth_weights: Q6_K needs a multiple of 256 elements");
    const int64_t nb = n_elements / 256; const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
    synth_q6_k_kernel<<<grid, 256, 0, s>>>((uint8_t*)out, nb, seed, amp);
  } else if (ggml_type == GGML_Q4_K) {
    TGA_REQUIRE(n_elements % 256 == 0, "tga_synth_weights: Q4_K needs a multiple of 256 elements");
    const int64_t nb = n_elements / 256; const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
    synth_q4_k_kernel<<<grid, 256, 0, s>>>((uint8_t*)out, nb, seed, amp);
  } else if (ggml_type == GGML_F16) {
    const int grid = (int)((n_elements + 255) / 256 < 65536 ? (n_elements + 255) / 256 : 65536);
    synth_f16_kernel<<<grid, 256, 0, s>>>((_Float16*)out, n_elements, seed, amp);
  } else if (ggml_type == GGML_MXFP4) {
    TGA_REQUIRE(n_elements % 32 == 0, "tga_synth_weights: MXFP4 needs a multiple of 32 elements");
    const int64_t nb = n_elements / 32; const int grid = (int)((nb + 255) / 256 < 65536 ? (nb + 255) / 256 : 65536);
    synth_mxfp4_kernel<<<grid, 256, 0, s>>>((uint8_t*)out, nb, seed, -8, -4);   // amp unused: exponents ~ U[-8, -4] (benchmark configuration 4)
  } else if (ggml_type == GGML_F32) {
    const int grid = (int)((n_elements + 255) / 256 < 65536 ? (n_elements + 255) / 256 : 65536);
    fill_f32_kernel<<<grid, 256, 0, s>>>((float*)out, n_elements, amp);   // constant fill (norm weights = 1)
  } else return tga_set_error("tga_synth_weights: unsupported type %d", ggml_type);
  TGA_LAUNCH_CHECK();
  return 0;
}
