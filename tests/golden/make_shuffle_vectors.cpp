// Writes tests/golden/column_sampling.json: the feature ids a tree may split on
// at every level, for a few (seed, columns, colsample_bytree, colsample_bylevel).
// Nothing here but the reference's calls on its random engine, in its order:
// engine(seed) once per booster (src/core/garden.cu:87), per tree ids 0..F-1
// and shuffle(all) (:142-146), per level shuffle(first int(bytree*F)) (:162-165),
// active = the first unsigned(bylevel*bytree*F) ids (:252-253, 309-310).
//   g++ -O1 -std=c++17 tests/golden/make_shuffle_vectors.cpp -o /tmp/msv && /tmp/msv > tests/golden/column_sampling.json
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>

int main() {
  struct Case { unsigned seed; size_t columns; float bytree, bylevel; int trees, levels; };
  const Case cases[] = {{0, 7, 0.5f, 1.0f, 3, 3},   {0, 28, 0.5f, 0.5f, 3, 4}, {5, 7, 1.0f, 0.6f, 2, 3},
                        {5, 28, 0.7f, 0.7f, 3, 4},  {0, 28, 1.0f, 1.0f, 2, 2}, {123, 12, 0.8f, 0.5f, 4, 5}};
  std::printf("[");
  for (const Case &c : cases) {
    std::default_random_engine rnd(c.seed);
    std::vector<unsigned int> active_fids(c.columns);
    std::printf("%s\n {\"seed\": %u, \"columns\": %zu, \"colsample_bytree\": %.9g, \"colsample_bylevel\": %.9g, \"active\": [",
                &c == cases ? "" : ",", c.seed, c.columns, c.bytree, c.bylevel);
    for (int t = 0; t < c.trees; ++t) {
      for (size_t i = 0; i < c.columns; ++i) active_fids[i] = i;
      std::shuffle(active_fids.begin(), active_fids.end(), rnd);
      std::printf("%s\n  [", t ? "," : "");
      for (int level = 0; level < c.levels; ++level) {
        int take = (int)(c.bytree * c.columns);
        std::shuffle(active_fids.begin(), active_fids.begin() + take, rnd);
        unsigned int active = (unsigned int)(c.bylevel * c.bytree * c.columns);
        std::printf("%s[", level ? ", " : "");
        for (unsigned j = 0; j < active; ++j) std::printf("%s%u", j ? ", " : "", active_fids[j]);
        std::printf("]");
      }
      std::printf("]");
    }
    std::printf("]}");
  }
  std::printf("\n]\n");
  return 0;
}
