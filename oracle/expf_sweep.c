/* TEST INFRASTRUCTURE ONLY.  Exhaustive check of oracle_expf_restated() against this
 * machine's libm expf over every float bit pattern (2^32 inputs, about a minute on 8
 * cores).  Prints the number of differing results (NaN payloads aside); exit code 0 iff
 * none differ.  Build: make -C oracle expf_sweep */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

float oracle_expf_restated(float x);

int main(void) {
  unsigned long long bad = 0;
  uint32_t first_bad = 0;
  /* touch once so that the table is built before the parallel region */
  (void)oracle_expf_restated(0.0f);
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (long long i = 0; i < (1LL << 32); ++i) {
    uint32_t u = (uint32_t)i;
    float x, a, b;
    memcpy(&x, &u, 4);
    a = expf(x);
    b = oracle_expf_restated(x);
    if (a != a && b != b) continue;
    if (memcmp(&a, &b, 4) != 0) {
      bad++;
      first_bad = u;
    }
  }
  printf("expf_sweep: %llu of 4294967296 inputs differ", bad);
  if (bad) printf(" (one of them: bits 0x%08x)", first_bad);
  printf("\n");
  return bad != 0;
}
