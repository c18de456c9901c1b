// Sample text -> resident shard, on the device.
//
// The reference's local_parser (alg/classification/logistic_regression/
// lr.cpp:76-93) turns every line "f1,f2,...,fk,label" into the sample
// [1.0, f1..fk] and its label with std::stod per field; for file-fed runs that
// parse, not the training pass, is what a worker waits for.  Here the worker's
// byte range of the input is copied to HBM as it is and parsed there:
//
//   csv_count_blocks  rows and fields that start in each 4 KiB block of text
//   csv_scan_blocks   their running sums (one workgroup): rows and fields in
//                     front of every block
//   csv_parse_fields  a workgroup per block, a lane per field
// (the three also run on one stretch of the text at a time, in text order, so
// that a stretch can be parsed while the next one is still on its way from the
// host: the running totals are carried in device memory from stretch to
// stretch)
//
// A field is converted on the device only when the result is provably strtod's,
// the correctly rounded value of the decimal.  The spelling must be
// [-]digits[.digits][e[+-]digits], with blanks or tabs in front if any and,
// behind a blank or tab (or the carriage return of a CR LF line end), anything
// at all -- what std::stod skips and what it ignores; then
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

// ---------------------------------------------------------------------------
// A lane per field.  A field belongs to the block its first character lies in,
// a row to the block its line starts in.  csv_count_blocks counts both per
// block, csv_scan_blocks turns the counts into "rows / fields in front of this
// block", and then every block is parsed on its own by one workgroup:
//   * the block (and the 64 bytes behind it) go to LDS with dense 16-byte loads
//     -- the text is read from memory once here, once by the count;
//   * every thread classifies its 16 bytes (terminators, field starts, line
//     starts), a prefix sum over the workgroup numbers the block's fields, and
//     the threads write the offsets of their field starts into a list in LDS;
//   * the fields of the list are dealt to the threads in turn: field k of the
//     block is field F + k of the text, i.e. (all lines holding d fields)
//     column (F + k) mod d of row (F + k) div d -- consecutive lanes convert
//     consecutive fields and store consecutive doubles of the shard;
//   * at every line start the number of fields in front of it must be d times
//     the number of rows in front of it; the first row for which it is not
//     names the ragged line (the host checks the last row against the total).
// Neither the length of a line nor the number of lines matters to the balance:
// 20001 fields a line or 3 parse at the same rate per byte.
struct CsvFieldArgs {
  const unsigned char* text;   // whole 4 KiB blocks, padded with '\n', + kCsvPadBytes
  const int64_t* first_row;    // per block: rows of the text in front of it
  const int64_t* first_field;  // per block: fields of the text in front of it
  int64_t block0;              // first block of this launch
  int64_t rows_cap;            // rows the shard holds: fields of later rows are dropped
  int d;                       // fields per line: k features, then the label
  unsigned char sep;
  double inv_d;                // 1.0 / d
  double* X;
  double* y;
  int64_t pitch;
  int np;                      // > 0: row-tiled layout with np column pairs per row
  CsvSlow* slow;
  int slow_cap;
  unsigned long long* slow_count;
  long long* bad_row;
};

// Field starts and line starts among 16 bytes of text (bit k = byte k); prev is
// the byte in front of them.  A field starts at a byte that is no terminator
// and follows one; a line starts at a byte that is no newline and follows one.
__device__ __forceinline__ void csv_classify16(const uint4 v, unsigned char prev, unsigned char sep,
                                               unsigned& fmask, unsigned& lmask) {
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  fmask = lmask = 0u;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const unsigned char ch = (unsigned char)(w[k >> 2] >> (8 * (k & 3)));
    const bool term = ch == sep || ch == '\n';
    const bool pterm = prev == sep || prev == '\n';
    if (!term && pterm) fmask |= 1u << k;
    if (ch != '\n' && prev == '\n') lmask |= 1u << k;
    prev = ch;
  }
}

// rows[b], fields[b] for the blocks block0 .. block0 + gridDim.x - 1
__global__ __launch_bounds__(kCsvThreads) void csv_count_blocks(const unsigned char* t,
                                                                unsigned char sep, int* rows,
                                                                int* fields, int64_t block0) {
  __shared__ int pr[kCsvThreads / 64], pf[kCsvThreads / 64];
  const int64_t blk = block0 + blockIdx.x;
  const int64_t base = (blk * kCsvThreads + threadIdx.x) * kCsvBytesPerThread;
  const uint4 v = *reinterpret_cast<const uint4*>(t + base);
  const unsigned char prev = base == 0 ? (unsigned char)'\n' : t[base - 1];
  unsigned fm, lm;
  csv_classify16(v, prev, sep, fm, lm);
  int cf = __builtin_popcount(fm), cr = __builtin_popcount(lm);
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    cf += __shfl_xor(cf, m, 64);
    cr += __shfl_xor(cr, m, 64);
  }
  if ((threadIdx.x & 63) == 0) {
    pf[threadIdx.x >> 6] = cf;
    pr[threadIdx.x >> 6] = cr;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int sf = 0, sr = 0;
    for (int w = 0; w < kCsvThreads / 64; ++w) {
      sf += pf[w];
      sr += pr[w];
    }
    fields[blk] = sf;
    rows[blk] = sr;
  }
}

// Running sums of rows[0..nblocks) and fields[0..nblocks) into first_row[] and
// first_field[] (what lies in front of each block), starting from totals[0]
// (rows) and totals[3] (fields) -- the text in front of these blocks -- and
// leaving the new totals there.  One workgroup.
__global__ __launch_bounds__(1024) void csv_scan_blocks(const int* rows, const int* fields,
                                                        int64_t nblocks, int64_t* first_row,
                                                        int64_t* first_field, int64_t* totals) {
  __shared__ int64_t wr[16], wf[16];
  __shared__ int64_t carry_r, carry_f;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) {
    carry_r = totals[0];
    carry_f = totals[3];
  }
  __syncthreads();
  for (int64_t i0 = 0; i0 < nblocks; i0 += 1024) {
    const int64_t i = i0 + threadIdx.x;
    const int64_t vr = i < nblocks ? rows[i] : 0, vf = i < nblocks ? fields[i] : 0;
    int64_t sr = vr, sf = vf;  // inclusive scans inside the wave
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
      const int64_t orr = __shfl_up(sr, m, 64), of = __shfl_up(sf, m, 64);
      if (lane >= m) {
        sr += orr;
        sf += of;
      }
    }
    if (lane == 63) {
      wr[wave] = sr;
      wf[wave] = sf;
    }
    __syncthreads();
    int64_t br = carry_r, bf = carry_f;
    for (int w = 0; w < wave; ++w) {
      br += wr[w];
      bf += wf[w];
    }
    if (i < nblocks) {
      first_row[i] = br + sr - vr;
      first_field[i] = bf + sf - vf;
    }
    __syncthreads();
    if (threadIdx.x == 1023) {
      carry_r = br + sr;
      carry_f = bf + sf;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    totals[0] = carry_r;
    totals[3] = carry_f;
  }
}

__global__ __launch_bounds__(kCsvThreads) void csv_parse_fields(CsvFieldArgs a) {
  constexpr int kAhead = 64;  // staged behind the block: 8 blanks, a number of 32 characters, its end
  static_assert(kAhead > 8 + kCsvMaxFieldChars + 2 && kAhead <= kCsvPadBytes, "look-ahead");
  __shared__ __align__(16) unsigned char txt[kCsvBlockBytes + kAhead];
  __shared__ unsigned short fpos[kCsvBlockBytes / 2 + 1];  // a field start at every other byte at most
  __shared__ int wf[kCsvThreads / 64], wr[kCsvThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t blk = a.block0 + blockIdx.x;
  const int64_t base = blk * kCsvBlockBytes;

  const uint4 mine = *reinterpret_cast<const uint4*>(a.text + base + tid * kCsvBytesPerThread);
  *reinterpret_cast<uint4*>(txt + tid * kCsvBytesPerThread) = mine;
  if (tid < kAhead / 16)
    *reinterpret_cast<uint4*>(txt + kCsvBlockBytes + tid * 16) =
        *reinterpret_cast<const uint4*>(a.text + base + kCsvBlockBytes + tid * 16);
  const unsigned char prev =
      (base == 0 && tid == 0) ? (unsigned char)'\n' : a.text[base + tid * kCsvBytesPerThread - 1];
  unsigned fm, lm;
  csv_classify16(mine, prev, a.sep, fm, lm);

  // fields and line starts in front of this thread's bytes, within the block
  const int nf = __builtin_popcount(fm), nl = __builtin_popcount(lm);
  int sf = nf, sl = nl;
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    const int of = __shfl_up(sf, m, 64), ol = __shfl_up(sl, m, 64);
    if (lane >= m) {
      sf += of;
      sl += ol;
    }
  }
  if (lane == 63) {
    wf[wave] = sf;
    wr[wave] = sl;
  }
  __syncthreads();
  int f0 = sf - nf, r0 = sl - nl, nfields = 0;
#pragma unroll
  for (int w = 0; w < kCsvThreads / 64; ++w) {
    if (w < wave) {
      f0 += wf[w];
      r0 += wr[w];
    }
    nfields += wf[w];
  }
  const int64_t blk_f0 = a.first_field[blk], blk_r0 = a.first_row[blk];

  // every line must hold d fields: in front of row r there are r * d of them
  {
    unsigned m = lm;
    int j = 0;
    while (m) {
      const int k = __builtin_ctz(m);
      m &= m - 1;
      const int64_t r = blk_r0 + r0 + j;
      const int64_t f = blk_f0 + f0 + __builtin_popcount(fm & ((1u << k) - 1u));
      if (f != r * (int64_t)a.d) atomicMin(a.bad_row, (long long)(r - 1));
      ++j;
    }
  }
  // this thread's field starts into the block's list
  {
    unsigned m = fm;
    int j = 0;
    while (m) {
      const int k = __builtin_ctz(m);
      m &= m - 1;
      fpos[f0 + j] = (unsigned short)(tid * kCsvBytesPerThread + k);
      ++j;
    }
  }
  __syncthreads();

  const int64_t fcap = a.rows_cap * (int64_t)a.d;
  for (int k = tid; k < nfields; k += kCsvThreads) {
    const int64_t f = blk_f0 + k;
    if (f >= fcap) continue;
    const int pos = fpos[k];
    // strtod's grammar for the exact spellings, a character per step.  The step
    // is straight-line code (selects, no branches): the lanes of a wave are at
    // different places of different fields, and every branch of an if-chain
    // would be walked by the whole wave.  A lane whose field has ended idles
    // until the longest field of the wave is through.
    unsigned long long m = 0;
    int sig = 0, ndig = 0, frac = 0, e10 = 0, ed = 0, st = 0, flen = 0;  // st: 0 int, 1 frac, 2 exp sign, 3 exp
    bool neg = false, eneg = false, bad = false, act = true;
    // std::stod skips white space in front of the number and ignores whatever
    // follows it.  White space in front (up to 8 characters) is passed over
    // before the walk; white space met during the walk -- a blank, a tab, the
    // carriage return of a CR LF line end -- ends the number like a terminator:
    // if it is complete by then (the checks behind the loop), the rest of the
    // field does not matter, and if not ("1e 5") the field is the host's, which
    // finds its end itself.
    auto blank = [](int ch) { return ch == ' ' || (unsigned)(ch - '\t') <= 4u; };  // isspace
    int lead = 0;
    while (lead < 8 && blank(txt[pos + lead]) && txt[pos + lead] != '\n' &&
           txt[pos + lead] != a.sep)  // (a separator may itself be a blank or a tab)
      ++lead;
    const int num = pos + lead;  // the number's first character
    bool blank_end = false;
    for (int j = 0; __any(act); ++j) {
      const int at = num + (act ? j : 0);
      const int ch = txt[at];
      const bool term = ch == a.sep || ch == '\n';
      // longer than the device converts: the host finds its end
      const bool over = act && !term && j == kCsvMaxFieldChars;
      bad = bad || over;
      flen = over ? -1 : flen;
      const bool stop = act && !term && !over && blank(ch);
      blank_end = blank_end || stop;
      act = act && !term && !over && !stop;
      const int dv = ch - '0';
      const bool digit = (unsigned)dv <= 9u;
      const bool mant = act && st <= 1;
      const bool mdig = mant && digit;
      m = mdig ? m * 10ull + (unsigned long long)dv : m;
      sig += (mdig && m != 0ull) ? 1 : 0;
      ndig += mdig ? 1 : 0;
      frac += (mdig && st == 1) ? 1 : 0;
      const bool minus0 = mant && ch == '-' && j == 0;
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
    }
    flen = (blank_end || flen < 0) ? -1 : flen + lead;  // as the host will read it, from pos
    if (e10 > 9999) bad = true;
    const int e = (eneg ? -e10 : e10) - frac;
    if (ndig == 0 || st == 2 || (st == 3 && ed == 0) || e < -44 || e > 44) bad = true;
    double v = 0.;
    if (!bad) {
      if (sig <= 15 && e >= -22 && e <= 22) {
        v = (double)m;
        v = e < 0 ? v / kCsvPow10[-e] : v * kCsvPow10[e];
      } else if (m != 0 && !csv_scale_dd(m, e, v)) {
        bad = true;
      }
    }
    // (row, column) of field f: f = row * d + col; the quotient by a reciprocal, corrected
    int64_t row = (int64_t)((double)f * a.inv_d);
    int64_t col = f - row * (int64_t)a.d;
    if (col < 0) {
      --row;
      col += a.d;
    } else if (col >= a.d) {
      ++row;
      col -= a.d;
    }
    if (!bad) {
      if (neg) v = -v;
      if (col == a.d - 1) {
        a.y[row] = v;
      } else if (a.np > 0) {
        a.X[((((row >> 6) * a.np + (col >> 1)) << 6) + (row & 63)) * 2 + (col & 1)] = v;
      } else {
        a.X[row * a.pitch + col] = v;
      }
    } else {
      const unsigned long long q = atomicAdd(a.slow_count, 1ull);
      if (q < (unsigned long long)a.slow_cap) {
        CsvSlow s;
        s.row = row;
        s.pos = base + pos;
        s.col = (int)col;
        s.len = flen;
        a.slow[q] = s;
      }
    }
  }
}

// values the host converted: X or y entries by flat index
__global__ void csv_patch(double* base, const int64_t* index, const double* value, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) base[index[i]] = value[i];
}

}  // namespace plr
