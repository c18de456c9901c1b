// Sample text -> resident shard, on the device.
//
// The reference's local_parser (alg/classification/logistic_regression/
// lr.cpp:76-93) turns every line "f1,f2,...,fk,label" into the sample
// [1.0, f1..fk] and its label with std::stod per field; for file-fed runs that
// parse, not the training pass, is what a worker waits for.  Here the worker's
// byte range of the input is copied to HBM as it is and parsed there:
//
//   csv_count_rows   line starts per 4 KiB block of text
//   csv_scan_counts  their running sum (one workgroup): first row of a block
//   csv_row_starts   byte offset of every row
// (these three and the parser also run on one stretch of the text at a time,
// in text order, so that a stretch can be parsed while the next one is still
// on its way from the host: the running row count is carried in device
// memory from stretch to stretch, and the parser reads its row range there)
//   csv_parse_rows   a lane per row, 64 rows per wave: every lane walks its own
//                    row through strtod's grammar (shards of many rows)
//   csv_parse        a wave per row: separators by ballot, one lane per field
//                    that starts in the wave's 64-byte window, the field's
//                    characters fetched from the neighbouring lanes (few rows)
//
// A field is converted on the device only when the result is provably strtod's,
// the correctly rounded value of the decimal.  The spelling must be
// [-]digits[.digits][e[+-]digits]; then
//   * at most 15 significant digits and a decimal exponent within +-22: the
//     digits are an exact double, 10^|e| is an exact double, and the one
//     multiplication or division rounds once (Clinger's fast path; the host
//     parser in worker/shard_io.hpp takes the same route);
//   * up to 19 significant digits (what "%.17g", repr() and "%.18e" write) and
//     an exponent within +-44: the digits, an exact 64-bit integer, are scaled
//     in double-double arithmetic (106 bits), and the result is taken only when
//     those 106 bits place the value clearly on one side of the nearest
//     rounding boundary -- anything closer than 2^-30 of a unit in the last
//     place to a tie, exact ties included, is left alone.
// Every other field is put on a list the host resolves with std::stod itself,
// so values and errors are the reference's for every input.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace plr {

constexpr int kCsvThreads = 256;
constexpr int kCsvBytesPerThread = 16;
constexpr int kCsvBlockBytes = kCsvThreads * kCsvBytesPerThread;  // 4 KiB
constexpr int kCsvMaxFieldChars = 32;  // longer fields go to the host
constexpr int kCsvPadBytes = 256;      // '\n' behind the text: a window may read past the end

// a field the device did not convert
struct CsvSlow {
  int64_t row;   // row of the shard
  int64_t pos;   // byte offset of the field's first character in the device text
  int32_t col;   // field index in the line (0 .. d-1; d-1 is the label)
  int32_t len;   // characters, or -1: longer than one window shows (the host finds its end)
};

struct CsvArgs {
  const unsigned char* text;  // len bytes followed by kCsvPadBytes of '\n'
  int64_t len;
  const int64_t* row_start;   // n byte offsets
  int64_t n;                  // rows of the shard (row_start, X, y hold that many)
  const int64_t* row_range;   // nullptr: parse rows 0 .. n-1; else the rows
                              //   row_range[0] .. min(row_range[1], n) - 1 (device memory)
  int d;                      // fields per line: k features, then the label
  unsigned char sep;
  double* X;                  // the shard: the k features of every row (the constant
  double* y;                  //   first column of the reference's sample is not stored)
  int64_t pitch;
  int np;                     // > 0: row-tiled layout with np column pairs per row
  CsvSlow* slow;
  int slow_cap;
  unsigned long long* slow_count;
  long long* bad_row;         // smallest row whose field count is not d
  int flush_at;               // csv_parse_rows: waiting fields that trigger their conversion
};

// line starts among the 16 bytes at `base` (a line starts after a newline, or
// at offset 0, and is not empty); their offsets go to out[] when given
__device__ __forceinline__ int csv_starts16(const unsigned char* t, int64_t base, int64_t len,
                                            int64_t* out) {
  if (base >= len) return 0;
  const uint4 v = *reinterpret_cast<const uint4*>(t + base);
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  unsigned char prev = base == 0 ? (unsigned char)'\n' : t[base - 1];
  int c = 0;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const unsigned char ch = (unsigned char)(w[k >> 2] >> (8 * (k & 3)));
    if (base + k < len && ch != '\n' && prev == '\n') {
      if (out) out[c] = base + k;
      ++c;
    }
    prev = ch;
  }
  return c;
}

// counts[b] for the blocks block0 .. block0 + gridDim.x - 1 of the text
__global__ __launch_bounds__(kCsvThreads) void csv_count_rows(const unsigned char* t, int64_t len,
                                                              int* counts, int64_t block0) {
  __shared__ int part[kCsvThreads / 64];
  const int64_t blk = block0 + blockIdx.x;
  const int64_t base = (blk * kCsvThreads + threadIdx.x) * kCsvBytesPerThread;
  int c = csv_starts16(t, base, len, nullptr);
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) c += __shfl_xor(c, m, 64);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int w = 0; w < kCsvThreads / 64; ++w) s += part[w];
    counts[blk] = s;
  }
}

// Running sum of counts[0..nblocks) into first_row[] (rows before each block),
// starting from *total (the rows of the text in front of these blocks) and
// leaving the new total there; range_out (nullable) receives the row range of
// these blocks, [old total, new total].
__global__ __launch_bounds__(1024) void csv_scan_counts(const int* counts, int64_t nblocks,
                                                        int64_t* first_row, int64_t* total,
                                                        int64_t* range_out) {
  __shared__ int64_t wsum[16];
  __shared__ int64_t carry_s;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) {
    carry_s = *total;
    if (range_out) range_out[0] = carry_s;
  }
  __syncthreads();
  for (int64_t i0 = 0; i0 < nblocks; i0 += 1024) {
    const int64_t i = i0 + threadIdx.x;
    const int64_t v = i < nblocks ? counts[i] : 0;
    int64_t s = v;  // inclusive scan inside the wave
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
      const int64_t o = __shfl_up(s, m, 64);
      if (lane >= m) s += o;
    }
    if (lane == 63) wsum[wave] = s;
    __syncthreads();
    int64_t before = carry_s;
    for (int w = 0; w < wave; ++w) before += wsum[w];
    if (i < nblocks) first_row[i] = before + s - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry_s = before + s;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    *total = carry_s;
    if (range_out) range_out[1] = carry_s;
  }
}

// row_start[] for the rows that start in blocks block0 .. block0 + gridDim.x - 1;
// rows at or past `cap` (the entries row_start holds) are not stored
__global__ __launch_bounds__(kCsvThreads) void csv_row_starts(const unsigned char* t, int64_t len,
                                                              const int64_t* first_row,
                                                              int64_t* row_start, int64_t block0,
                                                              int64_t cap) {
  __shared__ int part[kCsvThreads / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t blk = block0 + blockIdx.x;
  const int64_t base = (blk * kCsvThreads + threadIdx.x) * kCsvBytesPerThread;
  int64_t pos[kCsvBytesPerThread];
  const int c = csv_starts16(t, base, len, pos);
  int s = c;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    const int o = __shfl_up(s, m, 64);
    if (lane >= m) s += o;
  }
  if (lane == 63) part[wave] = s;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < wave; ++w) before += part[w];
  const int64_t at = first_row[blk] + before + s - c;
  for (int k = 0; k < c; ++k)
    if (at + k < cap) row_start[at + k] = pos[k];
}

// exact powers of ten
__device__ const double kCsvPow10[23] = {1e0,  1e1,  1e2,  1e3,  1e4,  1e5,  1e6,  1e7,
                                         1e8,  1e9,  1e10, 1e11, 1e12, 1e13, 1e14, 1e15,
                                         1e16, 1e17, 1e18, 1e19, 1e20, 1e21, 1e22};

// m * 10^e for 1 <= m < 2^64 and |e| <= 44, correctly rounded -- or false when
// 106 bits cannot tell on which side of a rounding boundary the value lies.
// The intrinsics keep every operation a single IEEE operation (no contraction).
__device__ __forceinline__ bool csv_scale_dd(unsigned long long m, int e, double& out) {
  // the integer as an unevaluated sum hi + lo of two doubles, exact
  double h = (double)m;  // round to nearest
  double l = (double)(long long)(m - (unsigned long long)h);  // |l| <= 2^10
  int left = e < 0 ? -e : e;
  while (left > 0) {
    const int k = left > 22 ? 22 : left;
    const double p = kCsvPow10[k];  // exact
    left -= k;
    double a, b;
    if (e < 0) {
      // (h + l) / p: quotient of the high part, its exact remainder, the correction
      a = __ddiv_rn(h, p);
      const double r = __dadd_rn(__fma_rn(-a, p, h), l);
      b = __ddiv_rn(r, p);
    } else {
      // (h + l) * p: product of the high part with its exact error, plus the low part's
      a = __dmul_rn(h, p);
      b = __dadd_rn(__fma_rn(h, p, -a), __dmul_rn(l, p));
    }
    h = __dadd_rn(a, b);                  // |b| << |a|: fast two-sum
    l = __dadd_rn(b, __dsub_rn(a, h));
  }
  // h is the value rounded to nearest unless hi + lo sits next to a tie: the
  // midpoint towards the neighbour on lo's side (below a power of two the
  // neighbour is half as far away)
  const long long hb = __double_as_longlong(h);  // h > 0
  const double nb = __longlong_as_double(l < 0. ? hb - 1 : hb + 1);
  const double half = __dmul_rn(0.5, fabs(__dsub_rn(nb, h)));
  const double off = fabs(__dsub_rn(fabs(l), half));
  if (off <= __dmul_rn(half, 9.313225746154785e-10)) return false;        // 2^-30
  out = h;
  return true;
}

__device__ __forceinline__ int csv_wave_max(int v) {
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    const int o = __shfl_xor(v, m, 64);
    v = o > v ? o : v;
  }
  return v;
}

__global__ __launch_bounds__(256) void csv_parse(CsvArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * 4;
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));  // lanes before mine
  const int64_t row_lo = a.row_range ? a.row_range[0] : 0;
  const int64_t row_hi = a.row_range ? (a.row_range[1] < a.n ? a.row_range[1] : a.n) : a.n;

  for (int64_t r = row_lo + wave0; r < row_hi; r += nwaves) {
    int64_t pos = a.row_start[r];
    int nfields = 0;       // fields of this row seen so far (uniform)
    bool prev_sep = true;  // the byte in front of the window ends a field (or the row starts here)
    bool done = false;
    while (!done) {
      // 128 bytes of the row: `cur` is this window, `nxt` the one behind it (the
      // text is padded with newlines, so both loads stay inside the buffer)
      const int cur = a.text[pos + lane];
      const int nxt = a.text[pos + 64 + lane];
      const unsigned long long nl_cur = __ballot(cur == '\n');
      const unsigned long long sep_cur = __ballot(cur == a.sep);
      const unsigned long long term_cur = nl_cur | sep_cur;
      const unsigned long long term_nxt = __ballot(nxt == '\n' || nxt == a.sep);
      const int endp = nl_cur ? __builtin_ctzll(nl_cur) : 64;  // the row's bytes are lanes < endp
      done = nl_cur != 0;
      // a field starts at a byte that is no terminator and follows one
      const bool after_term = lane == 0 ? prev_sep : ((term_cur >> (lane - 1)) & 1ull) != 0;
      const bool start = lane < endp && ((term_cur >> lane) & 1ull) == 0 && after_term;
      const unsigned long long start_mask = __ballot(start);
      int flen = 0;
      bool bad = false;
      if (start) {
        const unsigned long long t1 = lane == 63 ? 0ull : term_cur >> (lane + 1);
        if (t1)
          flen = 1 + __builtin_ctzll(t1);
        else if (term_nxt)
          flen = 64 - lane + __builtin_ctzll(term_nxt);
        else
          flen = -1;  // no end in sight
        if (flen < 0 || flen > kCsvMaxFieldChars) bad = true;
      }
      const int L = csv_wave_max((start && !bad) ? flen : 0);

      // strtod's grammar for the exact spellings, one character per step
      unsigned long long m = 0;
      int sig = 0, ndig = 0, frac = 0, e10 = 0, ed = 0, st = 0;  // st: 0 int, 1 frac, 2 exp sign, 3 exp
      bool neg = false, eneg = false;
      for (int j = 0; j < L; ++j) {
        const int src = lane + j;
        const int c0 = __shfl(cur, src & 63, 64);
        const int c1 = __shfl(nxt, src & 63, 64);
        const int ch = src < 64 ? c0 : c1;
        if (!start || bad || j >= flen) continue;
        const bool digit = ch >= '0' && ch <= '9';
        if (st <= 1) {
          if (digit) {
            m = m * 10ull + (unsigned long long)(ch - '0');
            if (m) ++sig;
            if (sig > 19) bad = true;  // 19 digits fit 64 bits
            ++ndig;
            if (st == 1) ++frac;
          } else if (ch == '-' && j == 0) {
            neg = true;
          } else if (ch == '.' && st == 0) {
            st = 1;
          } else if ((ch == 'e' || ch == 'E') && ndig > 0) {
            st = 2;
          } else {
            bad = true;
          }
        } else if (st == 2 && (ch == '+' || ch == '-')) {
          eneg = ch == '-';
          st = 3;
        } else if (digit) {
          st = 3;
          e10 = e10 * 10 + (ch - '0');
          if (e10 > 9999) bad = true;
          ++ed;
        } else {
          bad = true;
        }
      }

      if (start) {
        const int col = nfields + __builtin_popcountll(start_mask & below);
        int e = (eneg ? -e10 : e10) - frac;
        if (ndig == 0 || st == 2 || (st == 3 && ed == 0) || e < -44 || e > 44) bad = true;
        double v = 0.;
        if (!bad) {
          if (sig <= 15 && e >= -22 && e <= 22) {
            v = (double)m;
            v = e < 0 ? v / kCsvPow10[-e] : v * kCsvPow10[e];
          } else if (m == 0) {
            v = 0.;
          } else if (!csv_scale_dd(m, e, v)) {
            bad = true;
          }
        }
        if (col < a.d) {
          if (!bad) {
            if (neg) v = -v;
            if (col == a.d - 1) {
              a.y[r] = v;
            } else if (a.np > 0) {
              a.X[((((r >> 6) * a.np + (col >> 1)) << 6) + (r & 63)) * 2 + (col & 1)] = v;
            } else {
              a.X[r * a.pitch + col] = v;
            }
          } else {
            const unsigned long long k = atomicAdd(a.slow_count, 1ull);
            if (k < (unsigned long long)a.slow_cap) {
              CsvSlow s;
              s.row = r;
              s.pos = pos + lane;
              s.col = col;
              s.len = flen > kCsvMaxFieldChars ? -1 : flen;
              a.slow[k] = s;
            }
          }
        }
      }
      nfields += __builtin_popcountll(start_mask);
      prev_sep = ((term_cur >> 63) & 1ull) != 0;
      pos += 64;
    }
    if (nfields != a.d && lane == 0) atomicMin(a.bad_row, (long long)r);
  }
}

// The same parser with a lane per ROW: 64 consecutive rows per wave, every lane
// walking its own row 16 bytes at a time through strtod's grammar -- all 64
// lanes busy in the character step instead of the few that hold a field start.
// The conversion of a finished field (a division, the stores) is deferred: the
// field waits in a slot of its lane until most lanes have one waiting (or its
// lane finishes the next field), so that code runs once per several steps and
// with nearly every lane in it.
__global__ __launch_bounds__(256) void csv_parse_rows(CsvArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * 4;

  const int64_t row_lo = a.row_range ? a.row_range[0] : 0;
  const int64_t row_hi = a.row_range ? (a.row_range[1] < a.n ? a.row_range[1] : a.n) : a.n;

  for (int64_t r0 = row_lo + wave0 * 64; r0 < row_hi; r0 += nwaves * 64) {
    const int64_t r = r0 + lane;
    bool done = r >= row_hi;
    const int64_t start = done ? 0 : a.row_start[r];
    // the field in progress
    unsigned long long m = 0;
    int sig = 0, ndig = 0, frac = 0, e10 = 0, ed = 0, st = 0, flen = 0;
    bool neg = false, eneg = false, bad = false, infield = false;
    int col = 0;
    // the finished field waiting for its conversion
    bool pend = false, pneg = false, pbad = false;
    unsigned long long pm = 0;
    int pe = 0, psig = 0, pcol = 0, plen = 0;
    int64_t ppos = 0;

    auto flush = [&]() {
      if (pend) {
        double v = 0.;
        bool fb = pbad;
        if (!fb) {
          if (psig <= 15 && pe >= -22 && pe <= 22) {
            v = (double)pm;
            v = pe < 0 ? v / kCsvPow10[-pe] : v * kCsvPow10[pe];
          } else if (pm != 0 && !csv_scale_dd(pm, pe, v)) {
            fb = true;
          }
        }
        if (pcol < a.d) {
          if (!fb) {
            if (pneg) v = -v;
            if (pcol == a.d - 1) {
              a.y[r] = v;
            } else if (a.np > 0) {
              a.X[((((r >> 6) * a.np + (pcol >> 1)) << 6) + (r & 63)) * 2 + (pcol & 1)] = v;
            } else {
              a.X[r * a.pitch + pcol] = v;
            }
          } else {
            const unsigned long long k = atomicAdd(a.slow_count, 1ull);
            if (k < (unsigned long long)a.slow_cap) {
              CsvSlow s;
              s.row = r;
              s.pos = ppos;
              s.col = pcol;
              s.len = plen;
              a.slow[k] = s;
            }
          }
        }
        pend = false;
      }
    };

    // one character of this lane's row: `ch` at byte offset `at`
    auto step = [&](const int ch, const int64_t at) {
      const bool live = !done && at >= start;
      const bool term = ch == a.sep || ch == '\n';
      const bool closes = live && term && infield;
      // a lane about to finish a field while its slot is taken forces the conversions;
      // otherwise they wait until most lanes have one
      const unsigned long long waiting = __ballot(pend);
      if (__any(closes && pend) || __builtin_popcountll(waiting) >= a.flush_at) flush();
      // (everything below is straight-line code: selects, no branches)
      {
        const int e = (eneg ? -e10 : e10) - frac;
        const bool fbad = bad || ndig == 0 || st == 2 || (st == 3 && ed == 0) || e10 > 9999 ||
                          e < -44 || e > 44;
        pbad = closes ? fbad : pbad;
        pm = closes ? m : pm;
        pe = closes ? e : pe;
        psig = closes ? sig : psig;
        pneg = closes ? neg : pneg;
        pcol = closes ? col : pcol;
        plen = closes ? flen : plen;
        ppos = closes ? at - flen : ppos;
        pend = pend || closes;
        col += closes ? 1 : 0;
        infield = infield && !closes;
      }
      const bool ends = live && ch == '\n';
      if (__any(ends)) {
        if (ends && col != a.d) atomicMin(a.bad_row, (long long)r);
      }
      done = done || ends;
      // one character of the field
      const bool act = live && !term;
      const bool begin = act && !infield;
      m = begin ? 0ull : m;
      sig = begin ? 0 : sig;
      ndig = begin ? 0 : ndig;
      frac = begin ? 0 : frac;
      e10 = begin ? 0 : e10;
      ed = begin ? 0 : ed;
      st = begin ? 0 : st;
      flen = begin ? 0 : flen;
      neg = neg && !begin;
      eneg = eneg && !begin;
      bad = bad && !begin;
      infield = infield || act;
      const int dv = ch - '0';
      const bool digit = (unsigned)dv <= 9u;
      const bool mant = act && st <= 1;
      const bool mdig = mant && digit;
      m = mdig ? m * 10ull + (unsigned long long)dv : m;
      sig += (mdig && m != 0ull) ? 1 : 0;
      ndig += mdig ? 1 : 0;
      frac += (mdig && st == 1) ? 1 : 0;
      const bool minus0 = mant && ch == '-' && flen == 0;
      neg = neg || minus0;
      const bool dot = mant && ch == '.' && st == 0;
      const bool ee = mant && (ch | 0x20) == 'e' && ndig > 0;
      const bool esign = act && st == 2 && (ch == '+' || ch == '-');
      eneg = eneg || (esign && ch == '-');
      const bool edig = act && st >= 2 && digit;
      const int e_next = e10 * 10 + dv;
      e10 = edig ? (e_next > 99999 ? 99999 : e_next) : e10;
      ed += edig ? 1 : 0;
      bad = bad || (act && !(mdig || minus0 || dot || ee || esign || edig)) || sig > 19;
      st = dot ? 1 : ee ? 2 : (esign || edig) ? 3 : st;
      flen += act ? 1 : 0;
    };

    // A lane walks its row 16 bytes at a time; the chunk after the one being walked is
    // already on its way.  (Holding a whole 128-byte line per lane in registers, so that
    // no line is asked for twice, was measured: 15 % slower on 4.7 KB rows, 2.7 x slower
    // on 150-byte rows, whose neighbours share their lines.)
    int64_t chunk_at = start & ~(int64_t)15;
    uint4 nx = make_uint4(0x0a0a0a0au, 0x0a0a0a0au, 0x0a0a0a0au, 0x0a0a0a0au);
    if (!done) nx = *reinterpret_cast<const uint4*>(a.text + chunk_at);
    while (__any(!done)) {
      const uint4 v4 = nx;
      if (!done) nx = *reinterpret_cast<const uint4*>(a.text + chunk_at + 16);
      unsigned long long lo = ((unsigned long long)v4.y << 32) | v4.x;
      unsigned long long hi = ((unsigned long long)v4.w << 32) | v4.z;
#pragma clang loop unroll(disable)
      for (int k = 0; k < 16; ++k) {
        const int ch = (int)(lo & 0xffull);
        lo = (lo >> 8) | (hi << 56);
        hi >>= 8;
        step(ch, chunk_at + k);
      }
      chunk_at += 16;
    }
    flush();
  }
}

// values the host converted: X or y entries by flat index
__global__ void csv_patch(double* base, const int64_t* index, const double* value, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) base[index[i]] = value[i];
}

}  // namespace plr
