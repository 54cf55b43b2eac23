// Sanitizer driver of the CPU oracle (test infrastructure): compiled together with spconv_oracle.cpp under
// -fsanitize=address,undefined by `make -C oracle asan`, it calls every entry point on small seeded inputs that
// cover the shapes the tests use - SubM / strided / transposed rulebooks in 1 to 4 dims, truncated output
// capacity, capacity above the live count, an empty input; the three convolutions forward and inverse; the
// requantize rule; the voxeliser with rejected points; the dense map - so that an out-of-bounds access, a misaligned
// or overflowing operation ends the program.  It checks only what the sanitizers need to see plus a few
// invariants (-1 fill, 128-aligned count); values are the business of tests/test_oracle_pins.py.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

extern "C" {
uint32_t d3d_oracle_fmix32(uint32_t k);
void d3d_oracle_out_shape(int nd, const int32_t* inShape, const int32_t* k, const int32_t* s, const int32_t* p,
                          const int32_t* d, const int32_t* outPad, int transpose, int32_t* outShape);
int d3d_oracle_rulebook(int nd, const int32_t* coors, int32_t numActIn, int32_t cap, const int32_t* outShape,
                        const int32_t* k, const int32_t* s, const int32_t* p, const int32_t* d, int32_t maxNumActOut,
                        int subM, int transpose, int32_t* index, int32_t* numIndex, int32_t* outCoors,
                        int32_t* numActOut);
void d3d_oracle_conv_f32(const float* in, const float* w, const float* bias, const int32_t* index, int64_t rowLen,
                         int32_t numIndex, int cin, int cout, int32_t maxNumActOut, int inverse, int threads, float* out);
void d3d_oracle_conv_f64(const float* in, const float* w, const float* bias, const int32_t* index, int64_t rowLen,
                         int32_t numIndex, int cin, int cout, int32_t maxNumActOut, int inverse, int threads, double* out);
void d3d_oracle_conv_i8(const int8_t* in, const int8_t* w, const int32_t* index, int64_t rowLen, int32_t numIndex,
                        int cin, int cout, int32_t maxNumActOut, int inverse, int threads, int32_t* out);
void d3d_oracle_requantize(const int32_t* acc, const float* m, const float* bq, int64_t rows, int cout, int relu,
                           int8_t* out);
void d3d_oracle_bev_densify(const uint8_t* feats, const int32_t* coors, int32_t numActIn, int C, int elemBytes, int B,
                            int Z, int Y, int X, uint8_t* out);
int d3d_oracle_simple_mean(const float* feats, const int32_t* batchIdx, const float* config, int64_t numPts, int C,
                           int B, int Z, int Y, int X, int32_t maxNumActOut, float* outFeats, int32_t* outCoors,
                           int32_t* numActOut);
}

static uint64_t g_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd() {
  g_state = g_state * 6364136223846793005ull + 1442695040888963407ull;
  return static_cast<uint32_t>(g_state >> 33);
}
#define REQUIRE(c)                                                  \
  do {                                                              \
    if (!(c)) {                                                     \
      std::fprintf(stderr, "asan_check: %s (line %d)\n", #c, __LINE__); \
      std::exit(1);                                                 \
    }                                                               \
  } while (0)

// one rulebook + the three convolutions on it
static void runCase(int nd, const int* grid, int batch, int n, int cap, const int* k, const int* s, const int* p,
                    const int* d, int subM, int transpose, int maxOutScale) {
  std::vector<int32_t> coors(static_cast<size_t>(cap) * (nd + 1), 0);
  for (int i = 0; i < n; ++i) {  // duplicates are allowed: the oracle has to survive them
    coors[static_cast<size_t>(i) * (nd + 1)] = static_cast<int32_t>(rnd() % batch);
    for (int q = 0; q < nd; ++q) coors[static_cast<size_t>(i) * (nd + 1) + 1 + q] = static_cast<int32_t>(rnd() % grid[q]);
  }
  std::vector<int32_t> outPad(nd, 0), inShape(grid, grid + nd), outSpatial(nd);
  d3d_oracle_out_shape(nd, inShape.data(), k, s, p, d, outPad.data(), transpose, outSpatial.data());
  std::vector<int32_t> outShape(nd + 1);
  outShape[0] = batch;
  for (int q = 0; q < nd; ++q) outShape[1 + q] = subM ? grid[q] : outSpatial[q];
  int kVol = 1;
  for (int q = 0; q < nd; ++q) kVol *= k[q];
  const int64_t rowLen = static_cast<int64_t>(kVol) * (cap + 128);
  const int32_t maxOut = subM ? cap : (maxOutScale > 0 ? n * maxOutScale : n / 3 + 1);
  std::vector<int32_t> index(static_cast<size_t>(3 * rowLen), 7), outCoors(static_cast<size_t>(maxOut) * (nd + 1) + 1, 0);
  int32_t numIndex = -5, numActOut = -5;
  const int rc = d3d_oracle_rulebook(nd, coors.data(), n, cap, outShape.data(), k, s, p, d, maxOut, subM, transpose,
                                     index.data(), &numIndex, outCoors.data(), &numActOut);
  REQUIRE(rc == 0);
  REQUIRE(numIndex % 128 == 0 && numIndex >= 0 && numIndex <= rowLen);
  // (with no live input the oracle returns before its fills, as the reference does: trt/spconv/index.cu:271-275)
  for (int64_t i = numIndex; n > 0 && i < rowLen; ++i) REQUIRE(index[static_cast<size_t>(i)] == -1);
  if (!subM) REQUIRE(numActOut >= 0 && numActOut <= maxOut);
  const int cin = 5, cout = 7;
  const int32_t outRows = subM ? cap : maxOut, inRows = cap;
  for (int inverse = 0; inverse < 2; ++inverse) {
    const int32_t rowsIn = inverse ? outRows : inRows, rowsOut = inverse ? inRows : outRows;
    std::vector<float> in(static_cast<size_t>(rowsIn) * cin + 1), w(static_cast<size_t>(kVol) * cin * cout), bias(cout);
    for (auto& v : in) v = static_cast<float>(rnd() % 200) / 100.f - 1.f;
    for (auto& v : w) v = static_cast<float>(rnd() % 200) / 100.f - 1.f;
    for (auto& v : bias) v = 0.5f;
    std::vector<float> o32(static_cast<size_t>(rowsOut) * cout + 1);
    std::vector<double> o64(static_cast<size_t>(rowsOut) * cout + 1);
    d3d_oracle_conv_f32(in.data(), w.data(), bias.data(), index.data(), rowLen, numIndex, cin, cout, rowsOut, inverse, 2, o32.data());
    d3d_oracle_conv_f64(in.data(), w.data(), nullptr, index.data(), rowLen, numIndex, cin, cout, rowsOut, inverse, 1, o64.data());
    std::vector<int8_t> qi(static_cast<size_t>(rowsIn) * cin + 1), qw(static_cast<size_t>(kVol) * cin * cout);
    for (auto& v : qi) v = static_cast<int8_t>(rnd() % 255 - 127);
    for (auto& v : qw) v = static_cast<int8_t>(rnd() % 255 - 127);
    std::vector<int32_t> acc(static_cast<size_t>(rowsOut) * cout + 1);
    d3d_oracle_conv_i8(qi.data(), qw.data(), index.data(), rowLen, numIndex, cin, cout, rowsOut, inverse, 2, acc.data());
    std::vector<float> m(cout, 1e-3f), bq(cout, 0.25f);
    std::vector<int8_t> q(static_cast<size_t>(rowsOut) * cout + 1);
    d3d_oracle_requantize(acc.data(), m.data(), bq.data(), rowsOut, cout, inverse, q.data());
  }
}

int main() {
  REQUIRE(d3d_oracle_fmix32(0) == 0);
  const int one3[3] = {1, 1, 1}, two3[3] = {2, 2, 2}, k3[3] = {3, 3, 3}, zero3[3] = {0, 0, 0};
  const int grid3[3] = {9, 20, 18};
  runCase(3, grid3, 2, 500, 500, k3, one3, one3, one3, 1, 0, 0);       // SubM
  runCase(3, grid3, 2, 500, 700, k3, two3, one3, one3, 0, 0, 8);       // strided, capacity above the live count
  runCase(3, grid3, 1, 500, 500, k3, two3, one3, one3, 0, 0, -1);      // truncated output capacity
  runCase(3, grid3, 1, 300, 300, k3, two3, one3, one3, 0, 1, 27);      // transposed
  runCase(3, grid3, 1, 0, 256, k3, two3, one3, one3, 0, 0, 8);         // empty input
  runCase(3, grid3, 1, 0, 256, k3, one3, one3, one3, 1, 0, 0);
  const int k313[3] = {3, 1, 3}, p313[3] = {1, 0, 1};
  runCase(3, grid3, 1, 400, 400, k313, one3, p313, one3, 1, 0, 0);
  const int k311[3] = {3, 1, 1};
  runCase(3, grid3, 1, 400, 400, k311, two3, zero3, one3, 0, 0, 8);    // kernel (3,1,1), stride 2 everywhere
  runCase(3, grid3, 1, 300, 300, k3, one3, two3, two3, 1, 0, 0);       // dilation 2
  const int grid1[1] = {500}, k1[1] = {5}, s1[1] = {1}, p1[1] = {2}, d1[1] = {1};
  runCase(1, grid1, 2, 300, 300, k1, s1, p1, d1, 1, 0, 0);
  const int grid2[2] = {64, 64}, k2[2] = {3, 3}, s2[2] = {2, 2}, p2[2] = {1, 1}, d2[2] = {1, 1};
  runCase(2, grid2, 1, 700, 700, k2, s2, p2, d2, 0, 0, 4);
  const int grid4[4] = {6, 8, 10, 12}, k4[4] = {3, 3, 3, 3}, s4[4] = {1, 1, 1, 1}, p4[4] = {1, 1, 1, 1};
  runCase(4, grid4, 1, 600, 600, k4, s4, p4, s4, 1, 0, 0);

  // voxeliser: NaN / negative batch / out-of-grid points, a capacity below the voxel count
  {
    const int64_t nPts = 3000;
    const int C = 5, B = 2, Z = 4, Y = 30, X = 30;
    std::vector<float> feats(static_cast<size_t>(nPts) * C);
    std::vector<int32_t> batch(nPts);
    for (int64_t i = 0; i < nPts; ++i) {
      for (int c = 0; c < C; ++c) feats[static_cast<size_t>(i) * C + c] = static_cast<float>(rnd() % 4000) / 100.f - 5.f;
      batch[static_cast<size_t>(i)] = static_cast<int32_t>(rnd() % 4) - 1;  // -1 = skip, 2 = beyond B
    }
    feats[7] = 0.f / 1.f * __builtin_nanf("");
    const float config[6] = {0.f, 0.f, 0.f, 1.f, 1.f, 1.f};
    for (int32_t maxOut : {4000, 100}) {
      std::vector<float> outF(static_cast<size_t>(maxOut) * C);
      std::vector<int32_t> outC(static_cast<size_t>(maxOut) * 4), num(1);
      REQUIRE(d3d_oracle_simple_mean(feats.data(), batch.data(), config, nPts, C, B, Z, Y, X, maxOut, outF.data(),
                                     outC.data(), num.data()) == 0);
      REQUIRE(num[0] >= 0 && num[0] <= maxOut);
    }
  }
  // dense map, rows outside the grid included
  {
    const int n = 200, C = 3, B = 2, Z = 2, Y = 12, X = 10;
    for (int es : {1, 2, 4}) {
      std::vector<uint8_t> feats(static_cast<size_t>(n) * C * es, 1), out(static_cast<size_t>(B) * C * Z * Y * X * es);
      std::vector<int32_t> coors(static_cast<size_t>(n) * 4);
      for (int i = 0; i < n; ++i) {
        coors[static_cast<size_t>(i) * 4] = static_cast<int32_t>(rnd() % B);
        coors[static_cast<size_t>(i) * 4 + 1] = static_cast<int32_t>(rnd() % Z);
        coors[static_cast<size_t>(i) * 4 + 2] = static_cast<int32_t>(rnd() % Y);
        coors[static_cast<size_t>(i) * 4 + 3] = static_cast<int32_t>(rnd() % X);
      }
      d3d_oracle_bev_densify(feats.data(), coors.data(), n, C, es, B, Z, Y, X, out.data());
    }
  }
  std::puts("asan_check: ok");
  return 0;
}
