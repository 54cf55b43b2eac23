// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// CPU restatement of the sparse-convolution path of zhanggefan/deploy3d: the
// rulebook (index-pair) builder behind the SPConvIdx{1..4}d TensorRT plugins
// and the gather-GEMM-scatter behind SPConvMM.  The reference has no CPU path
// (trt/include/common/macros.h:58 is an empty tag); this file follows the
// CUDA implementation function by function, with serial loops where the
// reference races, so its output is one of the outputs the reference may
// legally produce.  Only tests/, the smoke check and the benchmark's
// cpu_baseline leg may load it; the shipped library never does.
//
// What pins each function (tests/test_oracle_pins.py, tests/test_golden.py):
//   out_shape      closed form; torch conv3d / conv_transpose3d output shapes
//   fmix32         published MurmurHash3 finaliser known answers
//   rulebook       brute-force dict rulebook on random clouds; the structural
//                  invariants held by the reference's own test
//                  (tests/spconv/test_spconv.py:72-124); dense-conv equivalence
//   conv_*         dense torch conv3d equivalence, 1x1x1 kernel == X @ W + b,
//                  single-voxel closed form, inverse == transposed adjacency
//   conv_i8/requant  integer exactness vs numpy int64; the requantize rule is
//                  NOT in the reference (trt/spconv/mm_trt.cu:184 accepts fp16
//                  only): parity unpinned by the reference, pinned only by the
//                  written rule restated above requantize() below.
//   simple_mean    torch unique + index_add scatter-mean, the formulation of the
//                  reference's own test (tests/voxel_encoder/test_simple_mean.py:17-33),
//                  on that test's two cases; truncation toward zero below the grid's
//                  minimum, NaN / negative-batch rows, the count under truncation
//   bev_densify    the dense-indexing ground truth of the reference's own test
//                  (tests/spconv/test_bev_densify.py:19-23) on its six cases
//
// Build: make -C oracle   (g++ -O2 -fopenmp -ffp-contract=off)
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace {

constexpr int kMaxDim = 4;
constexpr int kSegment = 128;  // TBSegment, trt/spconv/index.cu:21
constexpr int32_t kEmpty = std::numeric_limits<int32_t>::max();  // hash32.h:21

// trt/include/common/hash32.h:23-33 (Murmur3Hash4B)
inline uint32_t fmix32(uint32_t k) {
  k ^= k >> 16;
  k *= 0x85ebca6bu;
  k ^= k >> 13;
  k *= 0xc2b2ae35u;
  k ^= k >> 16;
  return k;
}

// trt/include/common/hash32.h:35-86 (LinearHashTable), executed serially.
struct LinearHash {
  std::vector<int32_t> keys, vals;
  size_t size;
  explicit LinearHash(size_t n) : keys(n, kEmpty), vals(n, 0), size(n) {}
  size_t insert(int32_t key, int32_t value) {  // hash32.h:59-71
    size_t slot = fmix32(uint32_t(key)) % size;
    for (size_t i = 0; i < size; i++) {
      if (keys[slot] == kEmpty || keys[slot] == key) {
        keys[slot] = key;
        vals[slot] = value;
        return slot;
      }
      slot = (slot + 1) % size;
    }
    return std::numeric_limits<size_t>::max();
  }
  bool lookup(int32_t key, int32_t& value) const {  // hash32.h:73-85
    size_t slot = fmix32(uint32_t(key)) % size;
    for (size_t i = 0; i < size; i++) {
      if (keys[slot] == key) {
        value = vals[slot];
        return true;
      }
      if (keys[slot] == kEmpty) return false;
      slot = (slot + 1) % size;
    }
    return false;
  }
};

// index.cu:209-213
size_t minPower2(size_t x) {
  size_t y = 1;
  while (y < x) y <<= 1;
  return y;
}

struct Geometry {
  int nd;
  int32_t k[kMaxDim], s[kMaxDim], p[kMaxDim], d[kMaxDim];
  int64_t shape[kMaxDim + 1];  // [B, spatial...]
  int kVol;
};

// refnd.h:33-39
inline bool isValid(const Geometry& g, const int32_t* c) {
  for (int i = 0; i <= g.nd; i++)
    if (c[i] < 0 || c[i] > g.shape[i] - 1) return false;
  return true;
}
// refnd.h:48-54
inline int64_t offsetOf(const Geometry& g, const int32_t* c) {
  int64_t off = c[0];
  for (int i = 1; i <= g.nd; i++) off = off * g.shape[i] + c[i];
  return off;
}
// refnd.h:56-64
inline void deserialize(const Geometry& g, int32_t* c, int64_t off) {
  for (int i = g.nd; i >= 0; i--) {
    c[i] = int32_t(off % g.shape[i]);
    off /= g.shape[i];
  }
}

// geometry.h:28-116.  Calls emit(tap, outCoor) for every tap of input voxel
// `in`, tap index row-major over the kernel dims; the forward form keeps only
// taps whose stride division is exact, the transposed form keeps all.
template <class Emit>
void forEachTap(const Geometry& g, const int32_t* in, bool transpose, Emit&& emit) {
  int32_t out[kMaxDim + 1];
  out[0] = in[0];  // geometry.h:105
  int idx[kMaxDim] = {0, 0, 0, 0};
  for (int tap = 0; tap < g.kVol; tap++) {
    bool ok = true;
    for (int dim = 0; dim < g.nd && ok; dim++) {
      if (transpose) {  // geometry.h:66-73
        out[dim + 1] = in[dim + 1] * g.s[dim] - g.p[dim] + idx[dim] * g.d[dim];
      } else {  // geometry.h:41-50; C++ % keeps the dividend's sign, so a
                // negative odd numerator is dropped and a negative even one
                // yields a negative coordinate that isValid() rejects
        int32_t c = in[dim + 1] + g.p[dim] - idx[dim] * g.d[dim];
        if (c % g.s[dim] != 0) ok = false;
        out[dim + 1] = c / g.s[dim];
      }
    }
    if (ok) emit(tap, out);
    for (int dim = g.nd - 1; dim >= 0; dim--) {  // row-major tap counter
      if (++idx[dim] < g.k[dim]) break;
      idx[dim] = 0;
    }
  }
}

// index.cu:123-156, 352-366: stable compaction of the [kVol, N] table,
// tap-major then input-row ascending, every tap segment starting on a
// multiple of 128; numIndex = end rounded up to 128.
void organize(const std::vector<int32_t>& table, int kVol, int64_t n, int64_t rowLen, int32_t* index,
              int32_t* numIndex) {
  int32_t* gather = index;
  int32_t* scatter = index + rowLen;
  int32_t* tapRow = index + 2 * rowLen;
  std::fill(index, index + 3 * rowLen, -1);  // index.cu:352-354, 459-461
  int64_t pos = 0;
  for (int k = 0; k < kVol; k++) {
    int64_t cnt = 0;
    for (int64_t i = 0; i < n; i++) {
      int32_t o = table[size_t(k) * n + i];
      if (o < 0) continue;
      gather[pos + cnt] = int32_t(i);
      scatter[pos + cnt] = o;
      tapRow[pos + cnt] = k;
      cnt++;
    }
    pos += (cnt + kSegment - 1) / kSegment * kSegment;
  }
  *numIndex = int32_t(pos);
}

Geometry makeGeometry(int nd, const int32_t* k, const int32_t* s, const int32_t* p, const int32_t* d,
                      const int32_t* outShape) {
  Geometry g{};
  g.nd = nd;
  g.kVol = 1;
  for (int i = 0; i < nd; i++) {
    g.k[i] = k[i];
    g.s[i] = s[i];
    g.p[i] = p[i];
    g.d[i] = d[i];
    g.kVol *= k[i];
  }
  for (int i = 0; i <= nd; i++) g.shape[i] = outShape[i];
  return g;
}

template <class In, class W, class Acc>
void convLoop(const In* in, const W* w, Acc* out, const int32_t* gather, const int32_t* scatter,
              const int32_t* tapRow, int64_t numIndex, int cin, int cout, int threads) {
  // test_spconv.py:152-161: for k: out[scatter[k]] += in[gather[k]] @ W[k].
  // Within one tap every scatter row appears at most once (one input maps to
  // one output per tap), so pairs of a tap segment are independent.
  int64_t j = 0;
  while (j < numIndex) {
    int32_t k = tapRow[j];
    if (k < 0) {  // padding slot (mm/kernel.h:100-101 exits on a padded tile)
      j++;
      continue;
    }
    int64_t e = j;
    while (e < numIndex && tapRow[e] == k) e++;
    const W* wk = w + size_t(k) * cin * cout;
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
    for (int64_t q = j; q < e; q++) {
      const In* x = in + size_t(gather[q]) * cin;
      Acc* y = out + size_t(scatter[q]) * cout;
      for (int ci = 0; ci < cin; ci++) {
        const Acc xv = Acc(x[ci]);
        const W* wr = wk + size_t(ci) * cout;
        for (int co = 0; co < cout; co++) y[co] += xv * Acc(wr[co]);
      }
    }
    j = e;
  }
}

}  // namespace

extern "C" {

uint32_t d3d_oracle_fmix32(uint32_t k) { return fmix32(k); }

// geometry.h:118-169 and index_trt.cu:128-150.  shapes are spatial only.
void d3d_oracle_out_shape(int nd, const int32_t* inShape, const int32_t* k, const int32_t* s, const int32_t* p,
                          const int32_t* d, const int32_t* outPad, int transpose, int32_t* outShape) {
  for (int i = 0; i < nd; i++) {
    if (transpose) {
      outShape[i] = (inShape[i] - 1) * s[i] - 2 * p[i] + (k[i] - 1) * d[i] + outPad[i] + 1;
    } else if (k[i] == -1) {
      outShape[i] = 1;
    } else {
      outShape[i] = (inShape[i] + 2 * p[i] - d[i] * (k[i] - 1) - 1) / s[i] + 1;
    }
  }
}

// createSparseSubMIndex (index.cu:400-476) and createSparseConvIndex
// (index.cu:253-368) behind SPConvIdxPlugin::enqueue (index_trt.cu:188-248).
//   coors     [cap, nd+1] int32 (b, spatial...), first numActIn rows live
//   outShape  [nd+1] = (B, spatial...) of the OUTPUT grid (SubM: input grid)
//   index     [3, kVol*(cap+128)]; numIndex [1]
//   outCoors  [maxNumActOut, nd+1], numActOut [1]   (conv only; may be null for SubM)
// Returns 0, or -1 on a full hash table (unreachable at load factor 1/2).
int d3d_oracle_rulebook(int nd, const int32_t* coors, int32_t numActIn, int32_t cap, const int32_t* outShape,
                        const int32_t* k, const int32_t* s, const int32_t* p, const int32_t* d, int32_t maxNumActOut,
                        int subM, int transpose, int32_t* index, int32_t* numIndex, int32_t* outCoors,
                        int32_t* numActOut) {
  Geometry g = makeGeometry(nd, k, s, p, d, outShape);
  const int64_t rowLen = int64_t(g.kVol) * (int64_t(cap) + kSegment);
  const int64_t n = numActIn;
  if (n == 0) {  // index.cu:271-275, 414-417: counts zeroed, index rows untouched
    *numIndex = 0;
    if (!subM && numActOut) *numActOut = 0;
    return 0;
  }
  const int cw = nd + 1;
  std::vector<int32_t> table(size_t(g.kVol) * n, -1);  // hashOut, 0xFF-filled (index.cu:309, 449)

  if (subM) {
    LinearHash hash(minPower2(size_t(n) * 2));  // index.cu:420
    for (int64_t i = 0; i < n; i++) hash.insert(int32_t(offsetOf(g, coors + i * cw)), int32_t(i));  // :174-182
    for (int64_t i = 0; i < n; i++) {  // subMGeometryKernel, index.cu:69-84, writer :48-66
      forEachTap(g, coors + i * cw, false, [&](int tap, const int32_t* o) {
        if (!isValid(g, o)) return;
        int32_t row;
        if (hash.lookup(int32_t(offsetOf(g, o)), row)) table[size_t(tap) * n + i] = row;
      });
    }
  } else {
    LinearHash hash(minPower2(size_t(g.kVol) * n * 2));  // index.cu:282
    std::vector<int64_t> slotOf(size_t(g.kVol) * n, -1);
    bool full = false;
    for (int64_t i = 0; i < n; i++) {  // convGeometryKernel, index.cu:86-102, writer :28-46
      forEachTap(g, coors + i * cw, transpose != 0, [&](int tap, const int32_t* o) {
        if (!isValid(g, o)) return;
        size_t slot = hash.insert(int32_t(offsetOf(g, o)), 1);
        if (slot == std::numeric_limits<size_t>::max()) full = true;
        slotOf[size_t(tap) * n + i] = int64_t(slot);
      });
    }
    if (full) return -1;
    // ExclusiveSum over hash values (index.cu:330-331) = rank in slot order
    std::vector<int32_t> unique(hash.size);
    int32_t run = 0;
    for (size_t sl = 0; sl < hash.size; sl++) {
      unique[sl] = run;
      run += hash.vals[sl];
    }
    // coorsOutOrganizeKernel (index.cu:104-121)
    for (size_t sl = 0; sl < hash.size; sl++) {
      if (hash.keys[sl] != kEmpty && unique[sl] < maxNumActOut)
        deserialize(g, outCoors + size_t(unique[sl]) * cw, hash.keys[sl]);
    }
    *numActOut = std::min(run, maxNumActOut);
    // hashOutIndexKernel (index.cu:158-172)
    for (size_t q = 0; q < table.size(); q++) {
      if (slotOf[q] < 0) continue;
      int32_t uid = unique[size_t(slotOf[q])];
      table[q] = uid < maxNumActOut ? uid : -1;
    }
  }
  organize(table, g.kVol, n, rowLen, index, numIndex);
  return 0;
}

// indexedSpConv (mm.h:35-71) + SPConvMMPlugin::enqueue (mm_trt.cu:149-205):
// every one of the maxNumActOut rows starts at the bias (mm.h:51-56), then the
// pair list is accumulated.  `inverse` swaps the gather and scatter rows
// (mm_trt.cu:174-177).  fp32 operands, fp32 accumulation.
void d3d_oracle_conv_f32(const float* in, const float* w, const float* bias, const int32_t* index, int64_t rowLen,
                         int32_t numIndex, int cin, int cout, int32_t maxNumActOut, int inverse, int threads,
                         float* out) {
  for (int64_t r = 0; r < maxNumActOut; r++)
    for (int c = 0; c < cout; c++) out[r * cout + c] = bias ? bias[c] : 0.f;
  const int32_t* gather = inverse ? index + rowLen : index;
  const int32_t* scatter = inverse ? index : index + rowLen;
  convLoop<float, float, float>(in, w, out, gather, scatter, index + 2 * rowLen, numIndex, cin, cout, threads);
}

// Same arithmetic with fp64 accumulation: the parity target for the fp32 and
// fp16 GPU kernels (fp16 operands are passed already rounded, as floats).
void d3d_oracle_conv_f64(const float* in, const float* w, const float* bias, const int32_t* index, int64_t rowLen,
                         int32_t numIndex, int cin, int cout, int32_t maxNumActOut, int inverse, int threads,
                         double* out) {
  for (int64_t r = 0; r < maxNumActOut; r++)
    for (int c = 0; c < cout; c++) out[r * cout + c] = bias ? double(bias[c]) : 0.0;
  const int32_t* gather = inverse ? index + rowLen : index;
  const int32_t* scatter = inverse ? index : index + rowLen;
  convLoop<float, float, double>(in, w, out, gather, scatter, index + 2 * rowLen, numIndex, cin, cout, threads);
}

// int8 operands, int32 accumulation, no bias (the bias enters at requantize).
void d3d_oracle_conv_i8(const int8_t* in, const int8_t* w, const int32_t* index, int64_t rowLen, int32_t numIndex,
                        int cin, int cout, int32_t maxNumActOut, int inverse, int threads, int32_t* out) {
  std::memset(out, 0, size_t(maxNumActOut) * cout * sizeof(int32_t));
  const int32_t* gather = inverse ? index + rowLen : index;
  const int32_t* scatter = inverse ? index : index + rowLen;
  convLoop<int8_t, int8_t, int32_t>(in, w, out, gather, scatter, index + 2 * rowLen, numIndex, cin, cout, threads);
}

// int8 requantize.  The reference has no int8 path; the rule is this build's:
//   t = (float)acc * m[c]      one fp32 multiply, no FMA contraction
//   t = t + bq[c]              one fp32 add
//   q = (int) rintf(t)         round-to-nearest-even
//   q = min(127, max(lo, q))   lo = 0 with fused ReLU, else -128
// with m[c] = (float)(s_in * s_w[c] / s_out), bq[c] = (float)(bias[c] / s_out)
// computed in double by the caller.  Compiled with -ffp-contract=off.
void d3d_oracle_requantize(const int32_t* acc, const float* m, const float* bq, int64_t rows, int cout, int relu,
                           int8_t* out) {
  const int lo = relu ? 0 : -128;
  for (int64_t r = 0; r < rows; r++) {
    for (int c = 0; c < cout; c++) {
      float t = float(acc[r * cout + c]) * m[c];
      t = t + bq[c];
      float q = rintf(t);  // clamped as a float so the int conversion never overflows
      q = std::fmin(127.f, std::fmax(float(lo), q));
      out[r * cout + c] = int8_t(int(q));
    }
  }
}

// kernel::densify after the memset (trt/spconv/bev_densify_trt.cu:22-35, :160-174): the map is [B, C, Z, Y, X],
// all zero except out[b, :, z, y, x] = feats[i, :] for every live row i with coordinate (b, z, y, x).  Rows are
// visited in order, so the last row naming a cell stays (the reference leaves that race open).  Elements are
// copied as bytes: elemBytes = 4 (float), 2 (half / bf16) or 1 (int8).
void d3d_oracle_bev_densify(const uint8_t* feats, const int32_t* coors, int32_t numActIn, int C, int elemBytes, int B,
                            int Z, int Y, int X, uint8_t* out) {
  const size_t plane = size_t(Z) * Y * X;
  std::memset(out, 0, size_t(B) * C * plane * elemBytes);
  for (int32_t i = 0; i < numActIn; i++) {
    const int32_t* c = coors + size_t(i) * 4;
    for (int ch = 0; ch < C; ch++) {
      const size_t at = (size_t(c[0]) * C + ch) * plane + (size_t(c[1]) * Y + c[2]) * X + c[3];
      std::memcpy(out + at * elemBytes, feats + (size_t(i) * C + ch) * elemBytes, elemBytes);
    }
  }
}

// simpleMeanEncoder (trt/voxel_encoder/simple_mean_trt.cu:26-168), executed serially in point order:
//   voxelize        (:28-60)  a point counts when all C features are finite, batch >= 0 and its cell
//                             (b, int((z-zMin)/zSize), int((y-yMin)/ySize), int((x-xMin)/xSize)) - fp32 arithmetic,
//                             conversion truncating toward zero - is inside the grid; the cell offset goes into a
//                             linear-probing table of 2*numPts slots (hash32.h:35-72), start slot fmix32(key) % size
//   inclusive scan  (:147-150) over the slots' occupancy: voxel id = scan - 1, so ids follow SLOT order;
//                             numActOut = min(occupied slots, maxNumActOut) (:87)
//   scatterAddFeats (:62-91)  ids below maxNumActOut accumulate feature sums and counts; the first point of a voxel
//                             writes its coordinate
//   meanFeats       (:93-101) rows below numActOut are divided by their count
// outFeats rows from numActOut on are zero (:142); outCoors rows from numActOut on are set to -1 here (the
// reference leaves them unwritten).  Returns 0, or -1 on a full table (cannot happen at load factor 1/2).
int d3d_oracle_simple_mean(const float* feats, const int32_t* batchIdx, const float* config, int64_t numPts, int C,
                           int B, int Z, int Y, int X, int32_t maxNumActOut, float* outFeats, int32_t* outCoors,
                           int32_t* numActOut) {
  const int64_t size = numPts * 2;
  std::vector<int64_t> key(size > 0 ? size : 1, -1);
  std::vector<int64_t> slotOf(numPts > 0 ? numPts : 1, -1);
  // float -> int32 as the device conversion does it: toward zero, saturating, NaN -> 0
  auto toInt = [](float v) -> int64_t {
    if (std::isnan(v)) return 0;
    if (v >= 2147483648.f) return 2147483647LL;
    if (v <= -2147483648.f) return -2147483648LL;
    return int64_t(int32_t(v));
  };
  for (int64_t i = 0; i < numPts; i++) {
    const float* f = feats + i * C;
    bool ok = true;
    for (int c = 0; c < C; c++) ok = ok && std::isfinite(f[c]);
    if (!ok) continue;
    const int64_t b = batchIdx[i];
    if (b < 0) continue;
    const int64_t x = toInt((f[0] - config[0]) / config[3]);
    const int64_t y = toInt((f[1] - config[1]) / config[4]);
    const int64_t z = toInt((f[2] - config[2]) / config[5]);
    if (b > B - 1 || z < 0 || z > Z - 1 || y < 0 || y > Y - 1 || x < 0 || x > X - 1) continue;
    const int64_t off = ((b * Z + z) * Y + y) * X + x;
    int64_t slot = int64_t(fmix32(uint32_t(off)) % uint64_t(size));
    int64_t tries = 0;
    for (; tries < size; tries++) {
      if (key[slot] == -1 || key[slot] == off) {
        key[slot] = off;
        slotOf[i] = slot;
        break;
      }
      slot = (slot + 1) % size;
    }
    if (tries == size) return -1;
  }
  std::vector<int32_t> scan(size > 0 ? size : 1, 0);
  int32_t run = 0;
  for (int64_t s = 0; s < size; s++) {
    run += key[s] != -1 ? 1 : 0;
    scan[s] = run;
  }
  *numActOut = run > maxNumActOut ? maxNumActOut : run;
  std::fill(outFeats, outFeats + int64_t(maxNumActOut) * C, 0.f);
  std::fill(outCoors, outCoors + int64_t(maxNumActOut) * 4, -1);
  std::vector<int32_t> count(maxNumActOut > 0 ? maxNumActOut : 1, 0);
  for (int64_t i = 0; i < numPts; i++) {
    const int64_t slot = slotOf[i];
    if (slot < 0) continue;
    const int32_t id = scan[slot] - 1;
    if (id >= maxNumActOut) continue;
    const int32_t firstOne = count[id]++;
    for (int c = 0; c < C; c++) outFeats[int64_t(id) * C + c] += feats[i * C + c];
    if (firstOne == 0) {
      int64_t off = key[slot];
      int32_t* row = outCoors + int64_t(id) * 4;
      row[3] = int32_t(off % X);
      off /= X;
      row[2] = int32_t(off % Y);
      off /= Y;
      row[1] = int32_t(off % Z);
      off /= Z;
      row[0] = int32_t(off);
    }
  }
  for (int32_t r = 0; r < *numActOut; r++)
    for (int c = 0; c < C; c++) outFeats[int64_t(r) * C + c] = outFeats[int64_t(r) * C + c] / float(count[r]);
  return 0;
}

}  // extern "C"
