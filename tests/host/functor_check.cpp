// Host-side check of a generated functor header: reads lines "s b h i j mq mk" from stdin and prints
// custom_score, custom_dscore and custom_keep for each.  Compiled with g++ by tests/test_compiler.py
// (-D__host__= -D__device__= -include <generated header>).
#include <cstdio>

int main() {
  double s;
  int b, h, i, j, mq, mk;
  while (std::scanf("%lf %d %d %d %d %d %d", &s, &b, &h, &i, &j, &mq, &mk) == 7) {
    std::printf("%.9g %.9g %d\n", (double)fa::custom_score((float)s, b, h, i, j, mq, mk),
                (double)fa::custom_dscore((float)s, b, h, i, j, mq, mk), fa::custom_keep(i, j) ? 1 : 0);
  }
  return 0;
}
