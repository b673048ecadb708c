// Host-side check of the 16-bit float conversions the kernels' epilogues use
// (iree_amd/csrc/uk_device.h, compiled here for the host) against the oracle's
// (oracle/uk_oracle.c, which restates common.h:665-792): every 16-bit input of
// the widening, and for the narrowing every sign, every f32 exponent field and
// every value of the mantissa bits that survive, each with the dropped bits at
// zero, one, just below a tie, the tie, just above it and all ones.
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "uk_device.h"

extern "C" {
float oracle_f16_to_f32(uint16_t h);
float oracle_bf16_to_f32(uint16_t h);
uint16_t oracle_f32_to_f16(float f);
uint16_t oracle_f32_to_bf16(float f);
}

static uint32_t bits_of(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float float_of(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

template <int EBITS>
static long check_narrow(uint16_t (*oracle)(float), const char* name) {
  const int shift = 23 - (15 - EBITS);
  const uint32_t half = 1u << (shift - 1), all = (1u << shift) - 1;
  const uint32_t low[6] = {0, 1, half - 1, half, half + 1, all};
  long bad = 0, count = 0;
  for (uint32_t top = 0; top < (1u << (32 - shift)); ++top)
    for (int l = 0; l < 6; ++l) {
      const uint32_t u = (top << shift) | low[l];
      const float f = float_of(u);
      const uint16_t want = oracle(f), got = uk::narrow16<EBITS>(f), steps = uk::narrow16_by_steps<EBITS>(f);
      ++count;
      if (got != want || steps != want) {
        if (bad++ < 8) printf("%s %08x: oracle %04x kernel %04x by steps %04x\n", name, u, want, got, steps);
      }
    }
  printf("%s: %ld inputs, %ld mismatches\n", name, count, bad);
  return bad;
}

int main() {
  long bad = 0;
  for (uint32_t h = 0; h < 65536; ++h) {
    if (bits_of(uk::widen16<5>((uint16_t)h)) != bits_of(oracle_f16_to_f32((uint16_t)h))) ++bad;
    if (bits_of(uk::widen16<8>((uint16_t)h)) != bits_of(oracle_bf16_to_f32((uint16_t)h))) ++bad;
  }
  printf("widen: %ld mismatches\n", bad);
  bad += check_narrow<5>(oracle_f32_to_f16, "f32->f16");
  bad += check_narrow<8>(oracle_f32_to_bf16, "f32->bf16");
  if (bad) return 1;
  printf("rounding check ok\n");
  return 0;
}
