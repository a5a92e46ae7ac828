/* Generator of viterbi_layout.h: the placement of trellis groups on the lanes of the Viterbi workgroup,
 * chosen by simulated annealing against a model of LDS bank conflicts.
 *
 *   cc -O2 -o gen_viterbi_layout gen_viterbi_layout.c -lm && ./gen_viterbi_layout [row_stride] [seed] [iters] > viterbi_layout.h
 *
 * Work split of the kernel.  Lane "unit" t = 2c + h (c = metric column 0..127, h = 0/1) owns, for every slot
 * m = 0..7, one of the two groups of column c whose low three bits are m:  j = 16c + 8 (h ^ s[c][m]) + m, and the
 * mirror group 4095 - j.  Free parameters: the bits s[c][m], which 16 units share a quarter-wave, and the padding
 * in front of each row of the error table.
 *
 * Model (measured on gfx950 with a ds_read_b64 microbenchmark: unit stride 4.4 cycles per wave access, stride of
 * two slots 8.2, random slots 11.9, all lanes on one bank pair 64): an 8-byte LDS access is served 16 lanes at a
 * time and each 16-lane quarter costs L cycles, L = the largest number of DISTINCT 8-byte addresses among its lanes
 * that fall on one of the 16 bank pairs.  Objective = modelled LDS cycles of one trellis step: error-table reads
 * (8 slots x 16 offsets), metric-column reads (2 x 16), metric writes (2 x 8).  The counter SQ_LDS_IDX_ACTIVE of the
 * real kernel follows this model to within 3 %.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int STRIDE = 33;
static int pad[64];
static uint8_t sel[128];     /* bit m: s[c][m] */
static int quarter[16][16];  /* unit ids */
static uint64_t rs = 88172645463325252ull;
static uint64_t rnd(void) {
  rs ^= rs << 13;
  rs ^= rs >> 7;
  rs ^= rs << 17;
  return rs;
}
static double rnd01(void) { return (rnd() >> 11) * (1.0 / 9007199254740992.0); }

static int group_of(int unit, int m) {
  int c = unit >> 1, h = unit & 1;
  return 16 * c + 8 * (h ^ ((sel[c] >> m) & 1)) + m;
}
static int maxload(const int* addr, int n) {
  int cnt[16] = {0}, best = 0;
  for (int i = 0; i < n; ++i) {
    int dup = 0;
    for (int k = 0; k < i; ++k)
      if (addr[k] == addr[i]) {
        dup = 1;
        break;
      }
    if (dup) continue;
    int b = ((addr[i] % 16) + 16) % 16;
    if (++cnt[b] > best) best = cnt[b];
  }
  return best;
}
static int cost_slot(const int* units, int m) {
  int e[16], wa[16], wb[16];
  for (int i = 0; i < 16; ++i) {
    int j = group_of(units[i], m), jb = 4095 - j;
    unsigned p = (unsigned)j * (unsigned)(j + 1);
    int row = (p >> 6) & 63, b4 = (p >> 12) & 15;
    e[i] = row * STRIDE + pad[row] + b4;
    wa[i] = (j & 255) * 17 + (j >> 8);
    wb[i] = (jb & 255) * 17 + (jb >> 8);
  }
  return 16 * maxload(e, 16) + maxload(wa, 16) + maxload(wb, 16);
}
static int cost_reads(const int* units) {
  int a[16], b[16];
  for (int i = 0; i < 16; ++i) {
    int c = units[i] >> 1;
    a[i] = c * 17;
    b[i] = (255 - c) * 17;
  }
  return 16 * maxload(a, 16) + 16 * maxload(b, 16);
}
static int cost_quarter(const int* units) {
  int t = cost_reads(units);
  for (int m = 0; m < 8; ++m) t += cost_slot(units, m);
  return t;
}

int main(int argc, char** argv) {
  if (argc > 1) STRIDE = atoi(argv[1]);
  if (argc > 2) rs ^= (uint64_t)atoll(argv[2]) * 0x9E3779B97F4A7C15ull;
  long iters = argc > 3 ? atol(argv[3]) : 30000000;
  int maxpad = STRIDE - 32;
  for (int q = 0; q < 16; ++q)
    for (int i = 0; i < 16; ++i) quarter[q][i] = 16 * q + i;
  int where_q[256], where_i[256];
  for (int q = 0; q < 16; ++q)
    for (int i = 0; i < 16; ++i) where_q[quarter[q][i]] = q, where_i[quarter[q][i]] = i;
  int qc[16], cur = 0;
  for (int q = 0; q < 16; ++q) cur += qc[q] = cost_quarter(quarter[q]);
  int start = cur, best = cur;
  int bpad[64], bquarter[16][16];
  uint8_t bsel[128];
  memcpy(bpad, pad, sizeof pad), memcpy(bsel, sel, sizeof sel), memcpy(bquarter, quarter, sizeof quarter);
  double T = 40.0;
  const double cool = pow(0.2 / 40.0, 1.0 / (double)iters);
  for (long it = 0; it < iters; ++it) {
    double r = rnd01();
    if (r < 0.45) { /* swap two units between quarters */
      int q1 = rnd() % 16, q2 = rnd() % 16;
      if (q1 == q2) continue;
      int i1 = rnd() % 16, i2 = rnd() % 16;
      int t = quarter[q1][i1];
      quarter[q1][i1] = quarter[q2][i2], quarter[q2][i2] = t;
      int c1 = cost_quarter(quarter[q1]), c2 = cost_quarter(quarter[q2]);
      int nw = cur - qc[q1] - qc[q2] + c1 + c2;
      if (nw <= cur || rnd01() < exp((cur - nw) / T)) {
        cur = nw, qc[q1] = c1, qc[q2] = c2;
        where_q[quarter[q1][i1]] = q1, where_i[quarter[q1][i1]] = i1;
        where_q[quarter[q2][i2]] = q2, where_i[quarter[q2][i2]] = i2;
      } else {
        t = quarter[q1][i1];
        quarter[q1][i1] = quarter[q2][i2], quarter[q2][i2] = t;
      }
    } else if (r < 0.9 || maxpad == 0) { /* flip which half of column c owns slot m */
      int c = rnd() % 128, m = rnd() % 8;
      int q1 = where_q[2 * c], q2 = where_q[2 * c + 1];
      sel[c] ^= (uint8_t)(1u << m);
      int c1 = cost_quarter(quarter[q1]), c2 = q2 == q1 ? c1 : cost_quarter(quarter[q2]);
      int nw = cur - qc[q1] - (q2 == q1 ? 0 : qc[q2]) + c1 + (q2 == q1 ? 0 : c2);
      if (nw <= cur || rnd01() < exp((cur - nw) / T)) {
        cur = nw, qc[q1] = c1;
        if (q2 != q1) qc[q2] = c2;
      } else {
        sel[c] ^= (uint8_t)(1u << m);
      }
    } else { /* move one row of the error table */
      int row = rnd() % 64, old = pad[row];
      pad[row] = rnd() % (maxpad + 1);
      int nqc[16], nw = 0;
      for (int q = 0; q < 16; ++q) nw += nqc[q] = cost_quarter(quarter[q]);
      if (nw <= cur || rnd01() < exp((cur - nw) / T)) {
        cur = nw;
        memcpy(qc, nqc, sizeof qc);
      } else {
        pad[row] = old;
      }
    }
    T *= cool;
    if (cur < best) {
      best = cur;
      memcpy(bpad, pad, sizeof pad), memcpy(bsel, sel, sizeof sel), memcpy(bquarter, quarter, sizeof quarter);
    }
    if (it % 5000000 == 0) fprintf(stderr, "it %ld cur %d best %d T %.2f\n", it, cur, best, T);
  }
  printf("// Generated by gen_viterbi_layout.c (row stride %d): modelled LDS cycles per trellis step %d\n", STRIDE, best);
  printf("// (identity placement %d, conflict-free bound 2816).\n", start);
  printf("//   kUnitOfLane[t]   unit 2c + h run by thread t (c: metric column, h: half)\n");
  printf("//   kHalfSel[c]      bit m set: the h = 0 unit of column c owns group 16c + 8 + m in slot m, else 16c + m\n");
  printf("//   kRowPad[r]       extra 8-byte slots in front of error-table row r (row stride %d)\n", STRIDE);
  printf("#pragma once\n#define QTIP_VIT_ROW_STRIDE %d\n", STRIDE);
  printf("__device__ const unsigned char kUnitOfLane[256] = {");
  for (int q = 0; q < 16; ++q)
    for (int i = 0; i < 16; ++i) printf("%d%s", bquarter[q][i], q == 15 && i == 15 ? "" : ",");
  printf("};\n__device__ const unsigned char kHalfSel[128] = {");
  for (int c = 0; c < 128; ++c) printf("%d%s", bsel[c], c == 127 ? "" : ",");
  printf("};\n__device__ const unsigned char kRowPad[64] = {");
  for (int r = 0; r < 64; ++r) printf("%d%s", bpad[r], r == 63 ? "" : ",");
  printf("};\n");
  return 0;
}
