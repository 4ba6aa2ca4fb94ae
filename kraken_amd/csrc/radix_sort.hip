// Stable least-significant-digit radix sort of (32-bit key, 32-bit payload) pairs on the device:
// what orders a large push's (row, position) pairs so that the gradient rows of one id are added
// up in position order (worker/emitter.cc:516-531 walks the request in order).
//
// A pass takes one digit of up to nine bits and is three launches with no waiting between
// workgroups:
//   1. radix_hist_kernel: every workgroup counts the digits of its tile of 4096 keys in LDS and
//      writes the counts digit-major, hist[digit][tile];
//   2. radix_scan_kernel: one wavefront per digit turns its row of counts into the number of
//      equal digits in earlier tiles, and notes the digit's total;
//   3. radix_scatter_kernel: a workgroup scans the 512 totals in LDS (where each digit's output
//      begins), ranks its tile's keys among equal digits in tile order (every wavefront finds the
//      lanes that hold the same digit with one ballot per digit bit, a per-wavefront histogram in
//      LDS turns into offsets by one scan over (digit, wavefront)), puts the tile into digit
//      order in LDS and writes it out from there, so that a digit's keys of the tile leave as one
//      piece: pair p of the ordered tile goes to begin[digit] + earlier[digit][tile] +
//      (p - where the digit starts in the tile).
// Equal digits keep their order in every pass, so the sort is stable.
#include "krk_internal.h"

namespace krk {

namespace {

constexpr int kRsBlock = 1024;
constexpr int kRsItems = 4;
constexpr int kRsTile = kRsBlock * kRsItems;     // keys a workgroup takes
constexpr int kRsWaves = kRsBlock / kWave;
constexpr int kRsMaxBits = 9;
constexpr int kRsDigits = 1 << kRsMaxBits;

// lanes of this wavefront (bit mask) whose `digit` equals this lane's
template <int BITS>
__device__ __forceinline__ unsigned long long same_digit(uint32_t digit) {
  unsigned long long same = ~0ull;
#pragma unroll
  for (int b = 0; b < BITS; ++b) {
    const bool bit = (digit >> b) & 1u;
    const unsigned long long votes = __ballot(bit);
    same &= bit ? votes : ~votes;
  }
  return same;
}

// lanes of this wavefront (bit mask) whose `digit` equals this lane's, for a digit of `bits` bits
__device__ __forceinline__ unsigned long long same_digit_n(uint32_t digit, int bits) {
  unsigned long long same = ~0ull;
  for (int b = 0; b < bits; ++b) {
    const bool bit = (digit >> b) & 1u;
    const unsigned long long votes = __ballot(bit);
    same &= bit ? votes : ~votes;
  }
  return same;
}

// Equal digits are counted once per wavefront: the lanes that hold the same digit find each
// other by votes and their first adds the group's size. (One LDS add per key serialises on the
// counter of a digit that many keys share: a request whose hottest row holds a quarter of the
// ids spent 5.9 us here per pass for a million keys, 11.8 us for two million.)
__global__ __launch_bounds__(kRsBlock) void radix_hist_kernel(const uint32_t* __restrict__ keys, int64_t n,
                                                              int shift, int bits, int64_t tiles,
                                                              uint32_t* __restrict__ hist) {
  __shared__ uint32_t count[kRsDigits];
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const uint32_t mask = (1u << bits) - 1u;
  if (t < kRsDigits) count[t] = 0u;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kRsTile;
  uint32_t key[kRsItems];
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    const int64_t j = base + i * kRsBlock + t;
    key[i] = j < n ? keys[j] : 0u;
  }
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    const bool live = base + i * kRsBlock + t < n;
    const uint32_t digit = (key[i] >> shift) & mask;
    const unsigned long long same = same_digit_n(digit, bits) & __ballot(live);
    if (live && (same & ((1ull << lane) - 1ull)) == 0ull) atomicAdd(&count[digit], (uint32_t)__popcll(same));
  }
  __syncthreads();
  if (t <= (int)mask) hist[(int64_t)t * tiles + blockIdx.x] = count[t];
}

// one wavefront per digit: hist[digit][0..tiles) -> exclusive prefix sums in place, total[digit]
__global__ __launch_bounds__(256) void radix_scan_kernel(uint32_t* __restrict__ hist, int64_t tiles, int digits,
                                                         uint32_t* __restrict__ total) {
  const int digit = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (digit >= digits) return;                         // the whole wavefront
  const int lane = threadIdx.x & (kWave - 1);
  uint32_t* row = hist + (int64_t)digit * tiles;
  uint32_t carry = 0;
  for (int64_t c0 = 0; c0 < tiles; c0 += kWave) {
    const int64_t c = c0 + lane;
    const uint32_t v = c < tiles ? row[c] : 0u;
    uint32_t incl = v;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    if (c < tiles) row[c] = carry + incl - v;
    carry += __shfl(incl, kWave - 1);
  }
  if (lane == 0) total[digit] = carry;
}

template <int BITS>
__global__ __launch_bounds__(kRsBlock) void radix_scatter_kernel(const uint32_t* __restrict__ keys,
                                                                 const uint32_t* __restrict__ vals, int64_t n,
                                                                 int shift, int64_t tiles,
                                                                 const uint32_t* __restrict__ hist,
                                                                 const uint32_t* __restrict__ total,
                                                                 uint32_t* __restrict__ keys_out,
                                                                 uint32_t* __restrict__ vals_out) {
  constexpr int kDigits = 1 << BITS;
  constexpr uint32_t kMask = kDigits - 1;
  __shared__ uint32_t gbase[kDigits];                  // where this tile's keys of the digit go in the output
  __shared__ uint32_t lstart[kDigits];                 // where they begin in the tile's own digit order
  __shared__ uint32_t wave_hist[kRsWaves * kDigits];   // [wave][digit]
  __shared__ uint32_t wave_total[kRsWaves];
  __shared__ uint32_t skey[kRsTile], sval[kRsTile];    // the tile in digit order
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  // element i of lane l in wavefront w is key w * 256 + i * 64 + l of the tile: a wavefront's
  // keys are consecutive, and taking i in ascending order visits them in tile order
  const int64_t tile_base = (int64_t)blockIdx.x * kRsTile;
  const int64_t base = tile_base + wave * (kWave * kRsItems) + lane;
  uint32_t key[kRsItems], val[kRsItems], rank[kRsItems];
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    const int64_t j = base + i * kWave;
    key[i] = j < n ? keys[j] : 0xFFFFFFFFu;
    val[i] = j < n ? vals[j] : 0u;
  }
  for (int i = t; i < kRsWaves * kDigits; i += kRsBlock) wave_hist[i] = 0u;
  // an exclusive scan over the workgroup's first kDigits lanes (one value each), through wave_total
  auto scan_digits = [&](uint32_t v) -> uint32_t {
    uint32_t incl = v;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    if (lane == kWave - 1) wave_total[wave] = incl;
    __syncthreads();
    uint32_t offset = incl - v;
    for (int w = 0; w < wave; ++w) offset += wave_total[w];
    return offset;
  };
  // where each digit's output begins (scan of the totals), plus what earlier tiles hold of it
  {
    const uint32_t offset = scan_digits(t < kDigits ? total[t] : 0u);   // its barrier: wave_hist is clear, too
    if (t < kDigits) gbase[t] = offset + hist[(int64_t)t * tiles + blockIdx.x];
  }
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    const bool live = base + i * kWave < n;            // the tile's tail holds no keys
    const uint32_t digit = (key[i] >> shift) & kMask;
    const unsigned long long same = same_digit<BITS>(digit) & __ballot(live);
    const uint32_t before = (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
    uint32_t* cell = &wave_hist[wave * kDigits + digit];
    const uint32_t old = *cell;                        // read by all lanes of the digit ...
    if (live && before == 0) *cell = old + (uint32_t)__popcll(same);   // ... then advanced by their first
    rank[i] = old + before;
  }
  __syncthreads();
  // per digit: what each wavefront holds of it becomes the count of the wavefronts before it,
  // and the digit's count in the tile goes on to the scan over digits (lane t owns digit t)
  uint32_t mine = 0;
  if (t < kDigits) {
#pragma unroll
    for (int w = 0; w < kRsWaves; ++w) {
      const uint32_t c = wave_hist[w * kDigits + t];
      wave_hist[w * kDigits + t] = mine;
      mine += c;
    }
  }
  {
    const uint32_t offset = scan_digits(mine);
    if (t < kDigits) lstart[t] = offset;
  }
  __syncthreads();
  // the tile in digit order, in LDS: equal digits keep their order
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    if (base + i * kWave < n) {
      const uint32_t digit = (key[i] >> shift) & kMask;
      const uint32_t at = lstart[digit] + wave_hist[wave * kDigits + digit] + rank[i];
      skey[at] = key[i];
      sval[at] = val[i];
    }
  }
  __syncthreads();
  // out: consecutive lanes hold consecutive keys of a digit, which go to consecutive addresses
  // (a digit's eight or so keys of a tile leave as one piece, not as eight)
  const int64_t left = n - tile_base;
  const int here = left < kRsTile ? (int)left : kRsTile;
#pragma unroll
  for (int i = 0; i < kRsItems; ++i) {
    const int p = i * kRsBlock + t;
    if (p < here) {
      const uint32_t k = skey[p];
      const uint32_t digit = (k >> shift) & kMask;
      const uint32_t dest = gbase[digit] + (uint32_t)p - lstart[digit];
      keys_out[dest] = k;
      vals_out[dest] = sval[p];
    }
  }
}

template <int BITS>
void launch_scatter(const uint32_t* keys, const uint32_t* vals, int64_t n, int shift, int64_t tiles,
                    const uint32_t* hist, const uint32_t* total, uint32_t* keys_out, uint32_t* vals_out,
                    hipStream_t stream) {
  hipLaunchKernelGGL((radix_scatter_kernel<BITS>), dim3((unsigned)tiles), dim3(kRsBlock), 0, stream, keys, vals, n,
                     shift, tiles, hist, total, keys_out, vals_out);
}

}  // namespace

size_t radix_sort_work_bytes(int64_t n) {
  const int64_t tiles = (n + kRsTile - 1) / kRsTile;
  return (size_t)(tiles + 1) * kRsDigits * sizeof(uint32_t);
}

int32_t radix_sort_pairs(uint32_t* keys, uint32_t* vals, uint32_t* keys_alt, uint32_t* vals_alt, int64_t n,
                         int bits, void* work, hipStream_t stream, uint32_t** keys_sorted,
                         uint32_t** vals_sorted) {
  if (bits < 1) bits = 1;
  if (bits > 32) bits = 32;
  const int64_t tiles = (n + kRsTile - 1) / kRsTile;
  if (tiles * (int64_t)kRsBlock >= ((int64_t)1 << 31)) {
    set_error("radix_sort_pairs: too many pairs for one launch");
    return KRK_E_CAPACITY;
  }
  uint32_t* hist = reinterpret_cast<uint32_t*>(work);
  uint32_t* total = hist + tiles * kRsDigits;
  const int passes = (bits + kRsMaxBits - 1) / kRsMaxBits;
  const int width = (bits + passes - 1) / passes;      // 8 or 9 bits where that saves nothing else
  uint32_t* src_k = keys;
  uint32_t* src_v = vals;
  uint32_t* dst_k = keys_alt;
  uint32_t* dst_v = vals_alt;
  for (int pass = 0; pass < passes && n > 0; ++pass) {
    const int shift = pass * width;
    const int w = bits - shift < width ? bits - shift : width;
    const int digits = 1 << w;
    hipLaunchKernelGGL(radix_hist_kernel, dim3((unsigned)tiles), dim3(kRsBlock), 0, stream, src_k, n, shift, w,
                       tiles, hist);
    hipLaunchKernelGGL(radix_scan_kernel, dim3((unsigned)((digits + 3) / 4)), dim3(256), 0, stream, hist, tiles,
                       digits, total);
    switch (w) {
      case 1: launch_scatter<1>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 2: launch_scatter<2>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 3: launch_scatter<3>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 4: launch_scatter<4>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 5: launch_scatter<5>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 6: launch_scatter<6>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 7: launch_scatter<7>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      case 8: launch_scatter<8>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
      default: launch_scatter<9>(src_k, src_v, n, shift, tiles, hist, total, dst_k, dst_v, stream); break;
    }
    KRK_HIP(hipGetLastError());
    uint32_t* tk = src_k;
    uint32_t* tv = src_v;
    src_k = dst_k;
    src_v = dst_v;
    dst_k = tk;
    dst_v = tv;
  }
  *keys_sorted = src_k;
  *vals_sorted = src_v;
  return KRK_SUCCESS;
}

}  // namespace krk
