// Deterministic synthetic voxel clouds and tensors for the sparse-convolution
// benchmarks and tests.  One implementation, used by the GPU harness, the
// benchmark driver and the fixture generator, so every consumer sees the same
// bits on every machine: splitmix64 streams, uniforms from the top 53 bits,
// normals by Box-Muller in fp64.
//
// Built as a plain host library (g++), no GPU code.
#include <cmath>
#include <cstdint>
#include <unordered_set>
#include <vector>

namespace {

struct SplitMix64 {
  uint64_t s;
  explicit SplitMix64(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  // uniform in [0,1) from the top 53 bits
  double uniform() { return double(next() >> 11) * (1.0 / 9007199254740992.0); }
  // floor(u*n), guaranteed < n
  int64_t below(int64_t n) {
    int64_t v = int64_t(uniform() * double(n));
    return v >= n ? n - 1 : v;
  }
  // Box-Muller, cosine branch only: two uniforms per normal, no cached state
  double normal() {
    double u1 = uniform(), u2 = uniform();
    return std::sqrt(-2.0 * std::log(1.0 - u1)) * std::cos(6.283185307179586476925286766559 * u2);
  }
};

inline int64_t linear(int64_t b, int64_t z, int64_t y, int64_t x, const int32_t* g) {
  return ((b * g[0] + z) * g[1] + y) * g[2] + x;
}

inline void put(int32_t* out, int64_t i, int b, int z, int y, int x) {
  out[4 * i + 0] = b;
  out[4 * i + 1] = z;
  out[4 * i + 2] = y;
  out[4 * i + 3] = x;
}

}  // namespace

extern "C" {

void d3d_synth_uniform_f64(uint64_t seed, double* out, int64_t n) {
  SplitMix64 r(seed);
  for (int64_t i = 0; i < n; i++) out[i] = r.uniform();
}

void d3d_synth_uniform_f32(uint64_t seed, float* out, int64_t n, double lo, double hi) {
  SplitMix64 r(seed);
  for (int64_t i = 0; i < n; i++) out[i] = float(lo + (hi - lo) * r.uniform());
}

void d3d_synth_normal_f32(uint64_t seed, float* out, int64_t n, double mean, double stddev) {
  SplitMix64 r(seed);
  for (int64_t i = 0; i < n; i++) out[i] = float(mean + stddev * r.normal());
}

uint64_t d3d_synth_splitmix64(uint64_t seed, int64_t nth) {
  SplitMix64 r(seed);
  uint64_t v = 0;
  for (int64_t i = 0; i <= nth; i++) v = r.next();
  return v;
}

// n unique voxels (b,z,y,x) whose linear offset is uniform over a
// [batch, grid[0], grid[1], grid[2]] grid; duplicates rejected, draw order kept.
// Returns the number written (n, or fewer if the grid has fewer cells).
int64_t d3d_synth_coords_uniform(uint64_t seed, int32_t batch, const int32_t* grid, int64_t n, int32_t* out) {
  SplitMix64 r(seed);
  const int64_t cells = int64_t(batch) * grid[0] * grid[1] * grid[2];
  if (n > cells) n = cells;
  std::unordered_set<int64_t> seen;
  seen.reserve(size_t(n) * 2);
  int64_t i = 0;
  while (i < n) {
    int64_t off = r.below(cells);
    if (!seen.insert(off).second) continue;
    int x = int(off % grid[2]);
    int64_t t = off / grid[2];
    int y = int(t % grid[1]);
    t /= grid[1];
    int z = int(t % grid[0]);
    int b = int(t / grid[0]);
    put(out, i++, b, z, y, x);
  }
  return n;
}

// Driving-scene LiDAR cloud, batch 1: the first floor(0.7 n) voxels lie on a
// ground shell (z uniform in {0..3}, y and x uniform); the rest fall in 200
// Gaussian clusters (centres uniform in the grid, sigma 3 in z and 8 in y/x,
// rounded to the nearest voxel).  Out-of-grid draws and duplicates are
// rejected; rows stay in draw order.
int64_t d3d_synth_coords_lidar(uint64_t seed, const int32_t* grid, int64_t n, int32_t* out) {
  SplitMix64 r(seed);
  std::unordered_set<int64_t> seen;
  seen.reserve(size_t(n) * 2);
  const int64_t nGround = (n * 7) / 10;
  const int zShell = grid[0] < 4 ? grid[0] : 4;
  int64_t i = 0;
  while (i < nGround) {
    int z = int(r.below(zShell));
    int y = int(r.below(grid[1]));
    int x = int(r.below(grid[2]));
    if (!seen.insert(linear(0, z, y, x, grid)).second) continue;
    put(out, i++, 0, z, y, x);
  }
  const int nClusters = 200;
  std::vector<int> cz(nClusters), cy(nClusters), cx(nClusters);
  for (int c = 0; c < nClusters; c++) {
    cz[c] = int(r.below(grid[0]));
    cy[c] = int(r.below(grid[1]));
    cx[c] = int(r.below(grid[2]));
  }
  while (i < n) {
    int c = int(r.below(nClusters));
    long z = cz[c] + std::lround(3.0 * r.normal());
    long y = cy[c] + std::lround(8.0 * r.normal());
    long x = cx[c] + std::lround(8.0 * r.normal());
    if (z < 0 || z >= grid[0] || y < 0 || y >= grid[1] || x < 0 || x >= grid[2]) continue;
    if (!seen.insert(linear(0, z, y, x, grid)).second) continue;
    put(out, i++, 0, int(z), int(y), int(x));
  }
  return n;
}

// Cylindrical segmentation cloud, batch 1, grid = [rho, phi, z]: rho is
// floor(Exp(mean 120)) clipped to the grid, phi uniform, z = round(N(8, 4))
// clipped to the grid.  Duplicates rejected, draw order kept.
int64_t d3d_synth_coords_cylinder(uint64_t seed, const int32_t* grid, int64_t n, int32_t* out) {
  SplitMix64 r(seed);
  std::unordered_set<int64_t> seen;
  seen.reserve(size_t(n) * 2);
  const int64_t cells = int64_t(grid[0]) * grid[1] * grid[2];
  if (n > cells) n = cells;
  int64_t i = 0;
  while (i < n) {
    double e = -120.0 * std::log(1.0 - r.uniform());
    long rho = long(std::floor(e));
    if (rho > grid[0] - 1) rho = grid[0] - 1;
    int phi = int(r.below(grid[1]));
    long z = std::lround(8.0 + 4.0 * r.normal());
    if (z < 0) z = 0;
    if (z > grid[2] - 1) z = grid[2] - 1;
    if (!seen.insert(linear(0, rho, phi, z, grid)).second) continue;
    put(out, i++, 0, int(rho), phi, int(z));
  }
  return n;
}

}  // extern "C"
