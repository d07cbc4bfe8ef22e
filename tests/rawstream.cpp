// Prints the raw stream of the construction-time generator the reference uses (src/rpucuda/rng.h:45-61,
// rng.cpp:21-31): ONE std::default_random_engine(seed), ONE persistent std::normal_distribution<float>{0,1}
// and ONE std::uniform_real_distribution<float>{0,1}.  It knows nothing about devices: the caller gives the
// order of the draws as a pattern string and assembles the expected arrays itself.
//   usage: rawstream <seed> <pattern> <repeats> [<threshold>]
//   pattern letters: N = one normal, U = one uniform,
//                    C = one uniform, and a second one if the first is below <threshold>
// Output: one line per draw, "<letter> <float as 8 hex digits>" (a second draw of C is tagged V).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

int main(int argc, char **argv) {
  if (argc < 4) return 2;
  std::default_random_engine gen((unsigned int)strtoul(argv[1], nullptr, 10));
  std::uniform_real_distribution<float> udist{0.0f, 1.0f};
  std::normal_distribution<float> ndist{0.0f, 1.0f};
  const char *pattern = argv[2];
  const long repeats = strtol(argv[3], nullptr, 10);
  const float threshold = argc > 4 ? strtof(argv[4], nullptr) : 0.0f;
  auto put = [](char tag, float v) {
    uint32_t bits;
    memcpy(&bits, &v, 4);
    printf("%c %08x\n", tag, bits);
  };
  for (long r = 0; r < repeats; ++r) {
    for (const char *c = pattern; *c; ++c) {
      if (*c == 'N') {
        put('N', ndist(gen));
      } else if (*c == 'U') {
        put('U', udist(gen));
      } else if (*c == 'C') {
        const float u = udist(gen);
        put('C', u);
        if (u < threshold) put('V', udist(gen));
      } else {
        return 3;
      }
    }
  }
  return 0;
}
