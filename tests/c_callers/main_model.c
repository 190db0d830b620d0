/* The application side of gen_model.c: the weights the generated file declares
 * extern, one call, the three results printed one per line
 * [ref: tests/compile/test_cxx_gen.in:51-68; expected output 6, 9, 12 at
 *  tests/compile/test_cxx_gen.cc:46-48]. */
#include <stdio.h>

const float w0[3] = {1, 2, 3}, w1[3] = {4, 5, 6};
extern int func(const float* in, float* out);
extern void func_fini(void);

int main(void) {
  float a[] = {1, 2, 3}, b[3] = {0, 0, 0};
  int s = func(a, b);
  if (s != 0) {
    printf("func failed: %d\n", s);
    return 1;
  }
  for (int i = 0; i < 3; ++i) printf("%f\n", b[i]);
  /* a second call reuses the computation and the context */
  a[0] = 10.f;
  if (func(a, b) != 0) return 1;
  printf("%f\n", b[0]);
  func_fini();
  return 0;
}
