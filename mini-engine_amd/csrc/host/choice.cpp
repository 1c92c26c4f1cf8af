// The choice of kernel per matrix product (see choice.h). The rules were measured on the layer sizes of a 0.6B, an 8B
// and a 32B model; the numbers stand beside them.
#include "choice.h"

#include "../kernels.h"

namespace me {

namespace {

constexpr int kF32 = 0, kBF16 = 1;
constexpr int kSmallFastRows = 16;  // up to here the small kernel beats the GEMM library on every shape, the norm as its prologue too
constexpr int kNormStreamRows = 2;  // up to here the add-and-norm is the prologue of the weight-streaming kernel
constexpr int kTiledMinRows = 256;
constexpr int kStreamWholeRows = 32;  // up to here the weight-streaming kernel serves wide plain products whose blocks fill whole
                                      // rounds (gated ones up to 64)
constexpr int kTiledMaxK = 3072;  // gate/up with the SwiGLU as the tiled kernel's epilogue against the library's product and a
                                  // SwiGLU kernel: at k = 1,024 (3,072 columns) 15-62 us against 21-67 for 512 to 4,096 rows; at
                                  // k = 4,096 (12,288 columns) 95-729 against 89-640; at k = 5,120 (25,600) 345-1,973 against
                                  // 293-1,767: the longer k is, the less a pass over the output weighs against the product
constexpr int kHeadStreamRows = 32;  // the head's logits (float32) come from the weight-streaming kernel up to here: at 151,936
                                     // rows of 1,024 / 4,096 / 5,120 it takes 62-75 / 245-272 / 291-341 us at 8 to 32 rows,
                                     // the library 62-79 / 260-276 / 319-362; from 48 rows on the library is ahead
constexpr int64_t kStreamMinElements = 8ll << 20;  // weights from 16 MiB on: streaming them is the product's time
constexpr int64_t kStreamMaxBytes = 1ll << 31;     // what the weight-streaming kernel addresses

// Which kernel serves a bfloat16 product of m rows:
//   up to 16 rows, weights below 16 MiB: the small matrix-core kernel; the residual add and the norm are its prologue
//     where the delta in front is a tensor (a product whose k was not cut);
//   17 to 64 rows, weights below 16 MiB: the weight-streaming kernel (qkv 5.0-6.7 us, gate/up with SwiGLU 6.6-9.3
//     against 5.8-7.7 and 7.5-10.3 with the small kernel, 8.2-8.6 and 14.4-14.7 with the library and a SwiGLU kernel);
//   a delta of the residual stream, at any row count up to 64: the weight-streaming kernel with k cut into runs, so
//     that every compute unit streams a part of the weight (1,024 columns, 1 to 16 rows: 3.5 and 4.3 us against 4.7-6.1
//     and 5.8-7.8 with the small kernel; 17 to 64 rows: 3.9-5.3 against 7.9-16 and 7.6-9.8). The add-and-norm behind
//     it, a kernel of its own (2.9 us), adds the partial sums up; as the prologue of the next product, where every
//     block would read them, they cost more at every row count (one row: 853 -> 820 tokens/s);
//   everything else: the GEMM library, as the reference hands every projection to one.
bool small_serves(int m, int k) { return k % 8 == 0 && m <= kSmallFastRows; }

// Whether a product of up to 64 rows is bound by streaming its weight: the layers of wide models. Their
// deltas go to the weight-streaming kernel with k cut into runs (measured at 4,096 and 5,120 columns, k of 4,096
// to 25,600: 8.7-29 us and 21-80 us against 9.4-65 and 27-245 with the small kernel, 10-38 and 20-156 with
// the library); their other products go to the same kernel up to 16 rows (qkv and gate/up 14.7-43 and 24-117 us
// against 15-51 and 26-139 with the small kernel) and to the library from 17 to 64 rows (qkv 15-33 us against
// 21-56 with the streaming kernel, whose time grows with the rows). The norm before such a product is a kernel
// of its own: the partial sums it adds up are read once, not by every block of a product.
bool weight_bound(int m, int rows_of_w, int k) {
  const int64_t elements = (int64_t)rows_of_w * k;
  return m <= kSmallMaxRows && k % 8 == 0 && elements >= kStreamMinElements && elements * 2 < kStreamMaxBytes;
}

// What the weight-streaming kernel takes in one group of rows.
bool streams(int m, int rows_of_w, int k) {
  return m <= kSmallMaxRows && k % 8 == 0 && (int64_t)rows_of_w * k * 2 < kStreamMaxBytes;
}

// Whether the weight-streaming kernel serves a wide product of 17 to 32 rows instead of the library: where its blocks fill
// whole rounds of the compute units (at least 15/16 of them) and the rows of the weight are a multiple of 4 KiB apart, which
// costs the library's kernels a quarter of their rate (2 x 12,288 x 4,096 with SwiGLU: 52 us, with k = 4,224 42; the streaming
// kernel 46 and 39). Measured at 17 and 32 rows: 2 x 12,288 x 4,096 46 us against 52; 6,144 x 4,096 14.1 and 15.6 against
// 16.3 and 15.9; 2 x 28,672 x 8,192 182 against 191 and 194; a decode step of the 8B shape at batch 20 to 32 4-5% shorter.
// Where the blocks do not fill their rounds the library is ahead (10,240 x 5,120 on 160 blocks: 32 and 35 against 27 and 30;
// 5,120 x 4,096: 13.4 against 12.0), with other k it is ahead or level (2 x 25,600 x 5,120: 101 and 105 against 99 and 102),
// and from 33 rows on it is ahead on as many shapes as not.
// With each block's walk over k starting at a step of its own (what the kernel does for such k) the gated products stay ahead
// up to 64 rows: 2 x 12,288 x 4,096 38-43 us against 48-50 at 17 to 64 rows, 2 x 14,336 x 4,096 45-48 against 58-65, 2 x 28,672
// x 8,192 169-180 against 192-216; the plain 6,144 x 4,096 up to 32 (14.3 and 15.1 against 15.1 and 15.4; 19.4 against 17.6 at 64).
// Plain products of weights between 16 and 32 MiB (the qkv of shapes between the narrow and the wide ones) stay with this
// kernel up to 32 rows whatever their k: 4,096 x 2,048 at 24 and 32 rows 8.2 us against 9.3 and 9.4 from the library, 6,144 x
// 2,560 10.5 and 11.3 against 11.6 and 11.9; from 48 rows on the two are level (9.6 and 9.4, 15.7 and 16.0).
bool stream_serves_mid_rows(int m, int n, int k, bool gated, int units) {
  if (!gated && m <= kStreamWholeRows && (int64_t)n * k < 2 * kStreamMinElements) return true;
  if (k % 2048 || m > (gated ? kSmallMaxRows : kStreamWholeRows)) return false;
  int plan[3] = {0, 0, 0};
  me_gemm_bf16_stream_plan(m, n, k, gated ? 1 : 0, 1, units, plan);
  const long long cus = units, rounds = (plan[2] + cus - 1) / cus;
  return (long long)plan[2] * 16 >= rounds * cus * 15;
}

}  // namespace

ProductChoice choose_product(int dtype, int role, int m, int rows_of_w, int k, int gated, int out_dtype, int units,
                             bool aligned) {
  ProductChoice c;
  const int n = gated ? rows_of_w / 2 : rows_of_w;
  if (dtype == kF32) {  // a true 32-bit product, additions in ascending k whatever the rows
    c.kernel = kProductF32;
    c.gate_after = gated != 0;
    return c;
  }
  const bool own = aligned && k % 8 == 0;  // what every kernel of this folder but the library's stand-ins needs
  if ((role == kRoleDelta || role == kRoleDeltaInto) && !gated) {
    c.partial_sums = true;
    if (own && streams(m, rows_of_w, k)) {
      // float32 partial sums over runs of k (one run for short k): the next add-and-norm adds them up, and the delta is
      // never rounded to bfloat16 on its way into the float32 residual stream
      c.kernel = kProductStream;
      c.runs = me_gemm_bf16_stream_splits(m, n, k, units);
      return c;
    }
    // More rows: the library's product with a float32 result. Where the caller can, the library adds it into the
    // residual stream in its own epilogue (x += product, a float32 sum per element), so that the norm behind reads
    // the stream alone and writes no new stream; else the result stands as one partial sum.
    c.kernel = kProductLibrary;
    if (role == kRoleDeltaInto && aligned && k % 8 == 0) {
      c.partial_sums = false;
      c.adds_into = true;
    }
    return c;
  }
  if (role == kRoleHead) {
    if (own && m > 2 && m <= kHeadStreamRows && weight_bound(m, rows_of_w, k))  // ahead of the small kernel and the library
      c.kernel = kProductStream;
    else if (own && m <= kSmallFastRows)
      c.kernel = kProductSmall;
    else
      c.kernel = kProductLibrary;
    return c;
  }
  const bool heavy = weight_bound(m, rows_of_w, k);
  const bool epilogue_fits = out_dtype == kBF16 || !gated;  // a gate's epilogue writes bfloat16
  if (own && epilogue_fits) {
    if (heavy && m <= kSmallFastRows) return c.kernel = kProductStream, c;  // up to 16 rows it is ahead of the library too
    if (heavy && stream_serves_mid_rows(m, n, k, gated != 0, units)) return c.kernel = kProductStream, c;
    if (!heavy && m > kSmallFastRows && streams(m, rows_of_w, k)) return c.kernel = kProductStream, c;
  }
  if (own && !heavy && small_serves(m, k)) return c.kernel = kProductSmall, c;
  if (own && gated && m <= kStreamGroupRows && (int64_t)rows_of_w * k < kStreamMinElements && out_dtype == kBF16) {
    // 65 to 256 rows of a small gated weight: the weight-streaming kernel, its blocks once per group of 64 rows (2 x 3,072 x
    // 1,024: 10.7-13.1 us against 15.5-19.1 with the library and a SwiGLU kernel, 16 with the tiled kernel; the plain
    // products of that size are no faster than the library's: 9.2 against 8.8-9.2, 7.8 against 7.6-8.3)
    return c.kernel = kProductStream, c;
  }
  if (gated && aligned && m >= kTiledMinRows && k % 64 == 0 && k <= kTiledMaxK && out_dtype == kBF16)
    return c.kernel = kProductTiled, c;  // ahead of the library product + SwiGLU kernel
  c.kernel = kProductLibrary;
  c.gate_after = gated != 0;
  return c;
}

// Decode-sized steps: the residual add and the norm are the product's prologue; the sum goes to the second residual
// buffer, since other blocks of the kernel still read the first.
// A row or two: the weight-streaming kernel adds and norms the rows itself while its first weights are on their way,
// whatever the delta is (one row: 857 -> 967 tokens/s, two: 1,605 -> 1,700; from four rows on every block's reads of
// the partial sums cost more than the launch they save: 2,749 -> 2,668; measured again with the prologue's loads requested
// together, against the carried norm below: three rows 1.289 -> 1.332 ms a step, four 1.371 -> 1.440; and the carried norm
// at two rows against this prologue: 1.157 -> 1.177).
// Up to 16 rows with nothing, or a tensor, to add (the first layer's norm; parts of other kinds): the small kernel's prologue.
int choose_norm_fusion(int dtype, int m, int rows_of_w, int k, int pending, int units, bool aligned) {
  (void)units;
  if (dtype != kBF16 || !aligned || k % 8) return kNormAlone;
  if (m <= kNormStreamRows && me_gemm_bf16_stream_norm_fits(m, k) && streams(m, rows_of_w, k)) return kNormInStream;
  if (m <= kSmallFastRows && pending != kPendingParts && !weight_bound(m, rows_of_w, k)) return kNormInSmall;
  return kNormAlone;
}

// From three rows on the add-and-norm is a kernel of its own (above), one of eight launches a layer whose floors are what a
// decode step of a few rows is made of. It goes away if the delta in front of it is summed over all of k by each block
// (no runs of k across blocks: a fourth as many blocks, each with a longer walk), which then adds its columns to the stream,
// writes bf16(x * w) and its part of the rows' sums of squares; the product behind the norm multiplies its rows by
// rsqrt(mean + eps). Measured on the same GPU in turns, layers of 1,024 x 2,048 (o), 1,024 x 3,072 (down), 4,096 and
// 2 x 3,072 x 1,024: the deltas take 6.7 us instead of 4.7 and the products behind them 0.6-0.9 more, the two add-and-norms
// (4.6 each under the profiler, about 3 inside a graph) are gone: a step of 3 / 4 / 8 items 1.246 -> 1.198 / 1.435 -> 1.387 /
// 1.778 -> 1.727 ms, of 10 / 12 / 16 items at a context of 2,048 1.604 -> 1.555 / 1.649 -> 1.599 / 1.844 -> 1.809. From 17 rows
// on (two tiles of rows a block) the whole-k deltas cost more than the launches they save (20 / 24 / 32 items: 1.97 -> 2.09 /
// 2.11 -> 2.24 / 1.81 -> 1.97 ms), and so they do on weights that take longer to stream than a launch costs (2,048 x 6,144 at 8
// rows: 10.7 us against 7.3 in runs; a step of the 32B shape at batch 8, whose 320 blocks of 16 columns are a round and a
// quarter of the compute units, 12% slower): up to 16 rows, weights below 16 MiB.
constexpr int kCarryMinRows = 3, kCarryMaxRows = 16;
bool choose_carried_norm(int dtype, int m, int n, int k, int next_rows_of_w, int next_gated, int units, bool aligned) {
  if (dtype != kBF16 || !aligned || m < kCarryMinRows || m > kCarryMaxRows || k % 8 || n % 8) return false;
  if (!streams(m, n, k) || (int64_t)n * k >= kStreamMinElements) return false;
  const ProductChoice next = choose_product(dtype, kRolePlain, m, next_rows_of_w, n, next_gated, dtype, units, aligned);
  return !next.gate_after && (next.kernel == kProductSmall || next.kernel == kProductStream);
}

// One item: a decode layer is six launches of about 5 us whose work is a fraction of that, and one of them only adds up the
// splits of attention. The output projection can do that at its head (me_attention_out_product_bf16), once per block of 64
// columns and run of heads: the splits' partial results are read as many times as the product has blocks of columns,
// which a narrow product bears (1,024 columns, 16 heads of 128, contexts of 1,024 / 2,304 / 4,096 / 8,192: a step of
// one item 1.027 -> 0.984 / 1.038 -> 1.001 / 1.042 -> 1.013 / 1.175 -> 1.106 ms; two items: 1.185 -> 1.202, the
// second row doubles what every block reads). Wider products are left to the two kernels: their blocks of columns would read
// more partial results than the product has weights (2,048 columns, the 1.7B shape's: a step of one item 1% longer).
constexpr int kSplitSumMaxRows = 1, kSplitSumMaxColumns = 1024;
bool choose_split_sum_in_product(int dtype, int m, int n, bool aligned) {
  return dtype == kBF16 && aligned && m <= kSplitSumMaxRows && n <= kSplitSumMaxColumns && n % 8 == 0;
}

}  // namespace me

// out: kernel, runs, partial_sums, gate_after, adds_into
extern "C" void me_product_choice(int dtype, int role, int m, int rows_of_w, int k, int gated, int out_dtype, int units,
                                  int aligned, int* out) {
  const me::ProductChoice c = me::choose_product(dtype, role, m, rows_of_w, k, gated, out_dtype, units, aligned != 0);
  out[0] = c.kernel;
  out[1] = c.runs;
  out[2] = c.partial_sums ? 1 : 0;
  out[3] = c.gate_after ? 1 : 0;
  out[4] = c.adds_into ? 1 : 0;
}

extern "C" int me_norm_fusion_choice(int dtype, int m, int rows_of_w, int k, int pending, int units, int aligned) {
  return me::choose_norm_fusion(dtype, m, rows_of_w, k, pending, units, aligned != 0);
}

extern "C" int me_carried_norm_choice(int dtype, int m, int n, int k, int next_rows_of_w, int next_gated, int units, int aligned) {
  return me::choose_carried_norm(dtype, m, n, k, next_rows_of_w, next_gated, units, aligned != 0) ? 1 : 0;
}

extern "C" int me_split_sum_choice(int dtype, int m, int n, int aligned) {
  return me::choose_split_sum_in_product(dtype, m, n, aligned != 0) ? 1 : 0;
}
