/* CPU oracle for the LLVQ fused dequant-GEMV path.  TEST INFRASTRUCTURE ONLY:
 * it may be called from tests, from the smoke test and from the benchmark's
 * CPU-baseline leg, never from the shipped library.
 *
 * Plain C restatement of the reference's CPU algorithm.  How each part is
 * pinned (tests/test_oracle_*.py):
 *   Golay table ............ weight enumerator 1+759x^8+2576x^12+759x^16+x^24,
 *                            (x+1) g1 g2 = x^23+1, distinctness, closure, and
 *                            every word folded into the fingerprint
 *   class enumeration ...... theta series m=2..5, closed form
 *                            65520/691 (sigma11 - tau) for m<=13, N(13), 383/301
 *                            classes, 3 classes on shell 2
 *   orc_index_decode ....... fingerprint 0x338f420f11866319
 *                            (llvq-artifact/tests/codebook_fingerprint.rs:58),
 *                            known-answer points, membership of every decoded
 *                            point, encode(decode(i)) = i, shell 2 and 3
 *                            exhaustive against an independent enumerator
 *   orc_fast_decode ........ equality with orc_index_decode on every class
 *                            boundary and on uniform draws (two independent
 *                            algorithms: factorial multinomials vs recurrence)
 *   bit stream ............. known answers of llvq-search/tests/g6_pack.rs
 *   matrix record .......... field order of format.rs:166-203, byte-identical
 *                            read->write passthrough, hostile-file cases
 *   reconstruct/decode ..... closed form; dense == fused to 1e-6 sum|wx|
 *   f16 conversions ........ all 65536 patterns against numpy
 *   SplitMix64 ............. published test vector for seed 0
 */
#include "llvq_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

typedef unsigned __int128 u128;

/* ======================================================================== */
/* Golay [24,12,8] — llvq-core/src/golay.rs                                  */
/* ======================================================================== */

#define GEN_POLY 0xC75u /* golay.rs:23 */

uint64_t orc_clmul(uint64_t a, uint64_t b) { /* golay.rs:32-42 */
  uint64_t acc = 0;
  while (b) {
    if (b & 1) acc ^= a;
    a <<= 1;
    b >>= 1;
  }
  return acc;
}

static uint32_t g_words[4096];
static int g_start[26]; /* g_start[w] .. g_start[w+1] = bucket of weight w */

static int popc(uint32_t v) { return __builtin_popcount(v); }

static int cmp_word(const void* a, const void* b) {
  uint32_t x = *(const uint32_t*)a, y = *(const uint32_t*)b;
  int px = popc(x), py = popc(y);
  if (px != py) return px < py ? -1 : 1;
  return x < y ? -1 : (x > y);
}

static void golay_build(void) { /* golay.rs:62-81 */
  for (uint32_t m = 0; m < 4096; m++) {
    uint32_t c = (uint32_t)orc_clmul(m, GEN_POLY);
    c |= (uint32_t)(popc(c) & 1) << 23;
    g_words[m] = c;
  }
  qsort(g_words, 4096, sizeof(uint32_t), cmp_word);
  memset(g_start, 0, sizeof g_start);
  for (int i = 0; i < 4096; i++) g_start[popc(g_words[i]) + 1]++;
  for (int w = 0; w < 25; w++) g_start[w + 1] += g_start[w];
}

/* ======================================================================== */
/* Classes — llvq-search/src/classes.rs, layout of index.rs:125-176           */
/* ======================================================================== */

#define MAX_CLASSES 512
#define MAX_SHELL 13

typedef struct {
  int shell, odd;
  /* even side */
  int w, p_req;
  int n_word, word_vals[4];
  uint8_t word_counts[4];
  int n_free, free_vals[4];
  uint8_t off_counts[8]; /* free counts, then the zero run (always present, may be 0) */
  int n_off;
  u128 a_on, a_off, s_w, s_f;
  /* odd side */
  int n_kinds, vals[8];
  uint8_t counts[8];
  u128 m_arr;
  /* layout */
  uint64_t offset, card;
  /* canonical levels, fastdec.rs:402-433 */
  int32_t lv_values[5];
  uint8_t lv_counts[5];
  int lv_len, lv_nonzero;
} cls_t;

static cls_t g_cls[MAX_CLASSES];
static int g_ncls;
static u128 g_fact[25];

static uint64_t gamma_w(int w) { /* classes.rs:35-44 */
  switch (w) {
    case 0: return 1;
    case 8: return 759;
    case 12: return 2576;
    case 16: return 759;
    case 24: return 1;
    default: return 0;
  }
}

static u128 multinomial(const uint8_t* counts, int k) { /* classes.rs:76-84 */
  int n = 0;
  for (int i = 0; i < k; i++) n += counts[i];
  u128 m = g_fact[n];
  for (int i = 0; i < k; i++) m /= g_fact[counts[i]];
  return m;
}

static void build_levels(cls_t* c, const int* v, const uint8_t* n, int k) {
  /* order: descending count, ties by descending value */
  int idx[8];
  for (int i = 0; i < k; i++) idx[i] = i;
  for (int i = 0; i < k; i++)
    for (int j = i + 1; j < k; j++) {
      int a = idx[i], b = idx[j];
      if (n[b] > n[a] || (n[b] == n[a] && v[b] > v[a])) {
        idx[i] = b;
        idx[j] = a;
      }
    }
  memset(c->lv_values, 0, sizeof c->lv_values);
  memset(c->lv_counts, 0, sizeof c->lv_counts);
  c->lv_len = k;
  c->lv_nonzero = 0;
  for (int i = 0; i < k && i < 5; i++) {
    c->lv_values[i] = v[idx[i]];
    c->lv_counts[i] = n[idx[i]];
    if (v[idx[i]] != 0) c->lv_nonzero += n[idx[i]];
  }
}

static cls_t e_tmp[MAX_CLASSES], o_tmp[MAX_CLASSES];

static void classes_build(void) {
  g_fact[0] = 1;
  for (int i = 1; i < 25; i++) g_fact[i] = g_fact[i - 1] * (u128)i;

  const int max_norm = 16 * MAX_SHELL;
  int ne = 0, no = 0;

  /* even: classes.rs:151-207 */
  for (int n14 = 0; n14 <= max_norm / 196; n14++)
    for (int n10 = 0; n10 <= max_norm / 100; n10++)
      for (int n6 = 0; n6 <= max_norm / 36; n6++)
        for (int n2 = 0; n2 <= max_norm / 4; n2++) {
          int w = n14 + n10 + n6 + n2;
          if (w > 24 || gamma_w(w) == 0) continue;
          int base = 196 * n14 + 100 * n10 + 36 * n6 + 4 * n2;
          if (base > max_norm) continue;
          for (int n12 = 0; n12 <= (max_norm - base) / 144; n12++)
            for (int n8 = 0; n8 <= (max_norm - base) / 64; n8++)
              for (int n4 = 0; n4 <= (max_norm - base) / 16; n4++) {
                int norm = base + 144 * n12 + 64 * n8 + 16 * n4;
                int total = w + n12 + n8 + n4;
                if (norm > max_norm || total > 24 || norm % 16 != 0) continue;
                int m = norm / 16;
                if (m < 2 || m > MAX_SHELL) continue;
                int s0 = 2 * n2 + 6 * n6 + 10 * n10 + 14 * n14 + 4 * n4 + 8 * n8 + 12 * n12;
                int p_req = (s0 / 4) % 2;
                if (w == 0 && p_req != 0) continue;
                cls_t* c = &e_tmp[ne++];
                memset(c, 0, sizeof *c);
                c->shell = m;
                c->w = w;
                c->p_req = p_req;
                const int wv[4] = {14, 10, 6, 2}, wn[4] = {n14, n10, n6, n2};
                for (int i = 0; i < 4; i++)
                  if (wn[i] > 0) {
                    c->word_vals[c->n_word] = wv[i];
                    c->word_counts[c->n_word++] = (uint8_t)wn[i];
                  }
                const int fv[3] = {12, 8, 4}, fn[3] = {n12, n8, n4};
                int free_n = 0;
                for (int i = 0; i < 3; i++)
                  if (fn[i] > 0) {
                    c->free_vals[c->n_free] = fv[i];
                    c->off_counts[c->n_free++] = (uint8_t)fn[i];
                    free_n += fn[i];
                  }
                int n0 = 24 - w - free_n;
                c->off_counts[c->n_free] = (uint8_t)n0;
                c->n_off = c->n_free + 1;
                c->a_on = multinomial(c->word_counts, c->n_word);
                c->a_off = multinomial(c->off_counts, c->n_off);
                c->s_w = w == 0 ? 1 : (u128)1 << (w - 1);
                c->s_f = (u128)1 << free_n;
                u128 card = (u128)gamma_w(w) * c->a_on * c->a_off * c->s_w * c->s_f;
                c->card = (uint64_t)card;
                int lv[8];
                uint8_t ln[8];
                int k = 0;
                for (int i = 0; i < c->n_word; i++) { lv[k] = c->word_vals[i]; ln[k++] = c->word_counts[i]; }
                for (int i = 0; i < c->n_free; i++) { lv[k] = c->free_vals[i]; ln[k++] = c->off_counts[i]; }
                if (n0 > 0) { lv[k] = 0; ln[k++] = (uint8_t)n0; }
                build_levels(c, lv, ln, k);
              }
        }

  /* odd: classes.rs:210-251 */
  for (int n13 = 0; n13 <= max_norm / 169; n13++)
    for (int n11 = 0; n11 <= max_norm / 121; n11++)
      for (int n9 = 0; n9 <= max_norm / 81; n9++)
        for (int n7 = 0; n7 <= max_norm / 49; n7++)
          for (int n5 = 0; n5 <= max_norm / 25; n5++) {
            int heavy = n13 + n11 + n9 + n7 + n5;
            if (heavy > 24) continue;
            int hnorm = 169 * n13 + 121 * n11 + 81 * n9 + 49 * n7 + 25 * n5;
            if (hnorm > max_norm) continue;
            for (int n3 = 0; n3 <= 24 - heavy; n3++) {
              int n1 = 24 - heavy - n3;
              int norm = hnorm + 9 * n3 + n1;
              if (norm > max_norm || norm % 16 != 0) continue;
              int m = norm / 16;
              if (m < 2 || m > MAX_SHELL) continue;
              if ((n1 + n7 + n9) % 2 != 1) continue;
              cls_t* c = &o_tmp[no++];
              memset(c, 0, sizeof *c);
              c->shell = m;
              c->odd = 1;
              const int ov[7] = {13, 11, 9, 7, 5, 3, 1}, on[7] = {n13, n11, n9, n7, n5, n3, n1};
              for (int i = 0; i < 7; i++)
                if (on[i] > 0) {
                  c->vals[c->n_kinds] = ov[i];
                  c->counts[c->n_kinds++] = (uint8_t)on[i];
                }
              c->m_arr = multinomial(c->counts, c->n_kinds);
              c->card = (uint64_t)((u128)4096 * c->m_arr);
              build_levels(c, c->vals, c->counts, c->n_kinds);
            }
          }

  /* layout: shells ascending, even then odd, enumeration order (index.rs:125-170) */
  g_ncls = 0;
  uint64_t off = 0;
  for (int m = 2; m <= MAX_SHELL; m++) {
    for (int i = 0; i < ne; i++)
      if (e_tmp[i].shell == m) g_cls[g_ncls++] = e_tmp[i];
    for (int i = 0; i < no; i++)
      if (o_tmp[i].shell == m) g_cls[g_ncls++] = o_tmp[i];
  }
  for (int i = 0; i < g_ncls; i++) {
    g_cls[i].offset = off;
    off += g_cls[i].card;
  }
  if (off != ORC_N13) abort(); /* index.rs:176 asserts the same */
}

static pthread_once_t g_once = PTHREAD_ONCE_INIT;
static void init_all(void) {
  golay_build();
  classes_build();
}
static void ensure_init(void) { pthread_once(&g_once, init_all); }

const uint32_t* orc_golay_codewords(void) {
  ensure_init();
  return g_words;
}
int orc_golay_of_weight(int w, const uint32_t** out) {
  ensure_init();
  if (w < 0 || w > 24) {
    if (out) *out = g_words;
    return 0;
  }
  if (out) *out = g_words + g_start[w];
  return g_start[w + 1] - g_start[w];
}
static int golay_rank_in_weight(uint32_t word) {
  int w = popc(word);
  if (w > 24) return -1;
  int lo = g_start[w], hi = g_start[w + 1];
  while (lo < hi) {
    int mid = (lo + hi) / 2;
    if (g_words[mid] < word) lo = mid + 1;
    else hi = mid;
  }
  if (lo < g_start[w + 1] && g_words[lo] == word) return lo - g_start[w];
  return -1;
}
int orc_golay_contains(uint32_t word) {
  ensure_init();
  return golay_rank_in_weight(word) >= 0;
}

static int rem_euclid(int64_t v, int64_t m) {
  int64_t r = v % m;
  return (int)(r < 0 ? r + m : r);
}

int orc_leech_contains(const int32_t x[ORC_DIM]) { /* leech.rs:76-99 */
  ensure_init();
  int p = rem_euclid(x[0], 2);
  for (int i = 0; i < ORC_DIM; i++)
    if (rem_euclid(x[i], 2) != p) return 0;
  uint32_t word = 0;
  for (int i = 0; i < ORC_DIM; i++)
    if (rem_euclid(((int64_t)x[i] - p) >> 1, 2) == 1) word |= 1u << i;
  if (!orc_golay_contains(word)) return 0;
  int64_t s = 0;
  for (int i = 0; i < ORC_DIM; i++) s += x[i];
  return rem_euclid(s, 8) == 4 * p;
}

int64_t orc_shell_index(const int32_t x[ORC_DIM]) { /* leech.rs:132-142 */
  int64_t n = 0;
  for (int i = 0; i < ORC_DIM; i++) n += (int64_t)x[i] * x[i];
  return n % 16 == 0 ? n / 16 : -1;
}

/* rng.rs:21-40 */
uint64_t orc_splitmix_next(uint64_t* s) {
  *s += 0x9E3779B97F4A7C15ULL;
  uint64_t z = *s;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}
double orc_splitmix_f64(uint64_t* s) {
  return (double)(orc_splitmix_next(s) >> 11) * (1.0 / 9007199254740992.0);
}
double orc_splitmix_gaussian(uint64_t* s) {
  double u1 = ((double)(orc_splitmix_next(s) >> 11) + 1.0) * (1.0 / 9007199254740993.0);
  double u2 = orc_splitmix_f64(s);
  return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
}

int orc_n_classes(void) {
  ensure_init();
  return g_ncls;
}
void orc_class_info(int ci, uint64_t* lo, uint64_t* hi, int* shell, int* odd, int* w,
                    int* n_levels) {
  ensure_init();
  const cls_t* c = &g_cls[ci];
  if (lo) *lo = c->offset + 1; /* fastdec.rs:301 */
  if (hi) *hi = c->offset + c->card;
  if (shell) *shell = c->shell;
  if (odd) *odd = c->odd;
  if (w) *w = c->w;
  if (n_levels) *n_levels = c->lv_len;
}
uint64_t orc_shell_cardinality(int m) {
  ensure_init();
  uint64_t s = 0;
  for (int i = 0; i < g_ncls; i++)
    if (g_cls[i].shell == m) s += g_cls[i].card;
  return s;
}
int orc_index_bits(uint32_t cap) { /* quantizer.rs:572-576 */
  ensure_init();
  uint64_t n = 0;
  for (uint32_t m = 2; m <= cap && m <= MAX_SHELL; m++) n += orc_shell_cardinality((int)m);
  int bits = n ? 64 - __builtin_clzll(n) : 0;
  return bits < 1 ? 1 : bits;
}
void orc_class_levels(int ci, int32_t values[5], uint8_t counts[5], int* len, int* nonzero) {
  ensure_init();
  const cls_t* c = &g_cls[ci];
  memcpy(values, c->lv_values, sizeof c->lv_values);
  memcpy(counts, c->lv_counts, sizeof c->lv_counts);
  if (len) *len = c->lv_len;
  if (nonzero) *nonzero = c->lv_nonzero;
}

/* ======================================================================== */
/* Indexer — llvq-search/src/index.rs                                         */
/* ======================================================================== */

/* index.rs:82-94 */
static u128 perm_rank(const uint8_t* kind_at, int n, uint8_t* counts, int k) {
  u128 rank = 0;
  for (int s = 0; s < n; s++) {
    int kk = kind_at[s];
    for (int j = 0; j < kk; j++)
      if (counts[j] > 0) {
        counts[j]--;
        rank += multinomial(counts, k);
        counts[j]++;
      }
    counts[kk]--;
  }
  return rank;
}

/* index.rs:97-117 */
static void perm_unrank(u128 rank, uint8_t* counts, int k, uint8_t* out, int n) {
  for (int s = 0; s < n; s++) {
    for (int j = 0; j < k; j++) {
      if (counts[j] == 0) continue;
      counts[j]--;
      u128 m = multinomial(counts, k);
      if (rank < m) {
        out[s] = (uint8_t)j;
        break;
      }
      rank -= m;
      counts[j]++;
    }
  }
}

static int find_class_linear(uint64_t i) { /* partition_point(offset+card <= i), index.rs:342-344 */
  int lo = 0, hi = g_ncls;
  while (lo < hi) {
    int mid = (lo + hi) / 2;
    if (g_cls[mid].offset + g_cls[mid].card <= i) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

int orc_index_decode(uint64_t idx, int32_t p[ORC_DIM]) { /* index.rs:334-435 */
  ensure_init();
  memset(p, 0, sizeof(int32_t) * ORC_DIM);
  if (idx == 0) return 1;
  uint64_t i = idx - 1;
  if (i >= ORC_N13) return 0;
  const cls_t* c = &g_cls[find_class_linear(i)];
  u128 local = (u128)(i - c->offset);
  if (!c->odd) {
    u128 r_sf = local % c->s_f; local /= c->s_f;
    u128 r_sw = local % c->s_w; local /= c->s_w;
    u128 r_off = local % c->a_off; local /= c->a_off;
    u128 r_on = local % c->a_on;
    size_t g = (size_t)(local / c->a_on);
    uint32_t cw = g_words[g_start[c->w] + g];
    int w = c->w;

    uint8_t wc[4], on_kinds[ORC_DIM];
    memcpy(wc, c->word_counts, 4);
    perm_unrank(r_on, wc, c->n_word, on_kinds, w);
    uint32_t sign[ORC_DIM] = {0}, par = 0;
    for (int j = 0; j + 1 < w; j++) {
      uint32_t b = (uint32_t)((r_sw >> j) & 1);
      sign[j] = b;
      par ^= b;
    }
    if (w > 0) sign[w - 1] = par ^ (uint32_t)c->p_req;
    int slot = 0;
    for (int q = 0; q < ORC_DIM; q++)
      if ((cw >> q) & 1) {
        int v = c->word_vals[on_kinds[slot]];
        p[q] = sign[slot] ? -v : v;
        slot++;
      }

    uint8_t oc[8], off_kinds[ORC_DIM];
    memcpy(oc, c->off_counts, 8);
    perm_unrank(r_off, oc, c->n_off, off_kinds, ORC_DIM - w);
    int zero_kind = c->n_free;
    slot = 0;
    int fbit = 0;
    for (int q = 0; q < ORC_DIM; q++)
      if (!((cw >> q) & 1)) {
        int k = off_kinds[slot];
        if (k != zero_kind) {
          int v = c->free_vals[k];
          p[q] = ((r_sf >> fbit) & 1) ? -v : v;
          fbit++;
        }
        slot++;
      }
  } else {
    u128 r_arr = local % c->m_arr;
    size_t g = (size_t)(local / c->m_arr);
    uint32_t cw = g_words[g];
    uint8_t counts[8], kinds[ORC_DIM];
    memcpy(counts, c->counts, 8);
    perm_unrank(r_arr, counts, c->n_kinds, kinds, ORC_DIM);
    for (int q = 0; q < ORC_DIM; q++) {
      int v = c->vals[kinds[q]];
      int a = (v % 4 == 3) ? v : -v;
      p[q] = ((cw >> q) & 1) ? a : -a;
    }
  }
  return 1;
}

int orc_index_encode(const int32_t x[ORC_DIM], uint64_t* out) { /* index.rs:190-330 */
  ensure_init();
  int allzero = 1;
  for (int i = 0; i < ORC_DIM; i++)
    if (x[i]) allzero = 0;
  if (allzero) { *out = 0; return 1; }
  if (!orc_leech_contains(x)) return 0;
  int64_t m = orc_shell_index(x);
  if (m < 2 || m > MAX_SHELL) return 0;
  int parity = rem_euclid(x[0], 2);
  uint32_t cw = 0;
  for (int i = 0; i < ORC_DIM; i++)
    if (rem_euclid(((int64_t)x[i] - parity) >> 1, 2) == 1) cw |= 1u << i;
  uint8_t cnt[16] = {0};
  for (int i = 0; i < ORC_DIM; i++) {
    int a = x[i] < 0 ? -x[i] : x[i];
    if (a > 15) return 0;
    cnt[a]++;
  }
  for (int ci = 0; ci < g_ncls; ci++) {
    const cls_t* c = &g_cls[ci];
    if (c->shell != m || c->odd != parity) continue;
    uint8_t sig[16] = {0};
    if (!c->odd) {
      for (int i = 0; i < c->n_word; i++) sig[c->word_vals[i]] = c->word_counts[i];
      for (int i = 0; i < c->n_free; i++) sig[c->free_vals[i]] = c->off_counts[i];
      sig[0] = cnt[0];
    } else {
      for (int i = 0; i < c->n_kinds; i++) sig[c->vals[i]] = c->counts[i];
    }
    if (memcmp(sig, cnt, 16)) continue;

    u128 local;
    if (!c->odd) {
      int g = golay_rank_in_weight(cw);
      if (g < 0) return 0;
      uint8_t on_kinds[ORC_DIM], off_kinds[ORC_DIM];
      uint32_t sbits[ORC_DIM];
      int n_on = 0, n_offs = 0, nfb = 0;
      u128 r_sf = 0;
      for (int i = 0; i < ORC_DIM; i++) {
        int a = x[i] < 0 ? -x[i] : x[i];
        if ((cw >> i) & 1) {
          int k = -1;
          for (int j = 0; j < c->n_word; j++)
            if (c->word_vals[j] == a) k = j;
          if (k < 0) return 0;
          on_kinds[n_on] = (uint8_t)k;
          sbits[n_on++] = x[i] < 0;
        } else if (x[i] == 0) {
          off_kinds[n_offs++] = (uint8_t)c->n_free;
        } else {
          int k = -1;
          for (int j = 0; j < c->n_free; j++)
            if (c->free_vals[j] == a) k = j;
          if (k < 0) return 0;
          off_kinds[n_offs++] = (uint8_t)k;
          if (x[i] < 0) r_sf |= (u128)1 << nfb;
          nfb++;
        }
      }
      uint8_t wc[4], oc[8];
      memcpy(wc, c->word_counts, 4);
      memcpy(oc, c->off_counts, 8);
      u128 r_on = perm_rank(on_kinds, n_on, wc, c->n_word);
      u128 r_off = perm_rank(off_kinds, n_offs, oc, c->n_off);
      u128 r_sw = 0;
      for (int j = 0; j + 1 < c->w; j++) r_sw |= (u128)sbits[j] << j;
      local = ((((u128)g * c->a_on + r_on) * c->a_off + r_off) * c->s_w + r_sw) * c->s_f + r_sf;
    } else {
      int w = popc(cw);
      int gi = golay_rank_in_weight(cw);
      if (gi < 0) return 0;
      gi += g_start[w];
      uint8_t kinds[ORC_DIM], counts[8];
      for (int i = 0; i < ORC_DIM; i++) {
        int a = x[i] < 0 ? -x[i] : x[i];
        int k = -1;
        for (int j = 0; j < c->n_kinds; j++)
          if (c->vals[j] == a) k = j;
        if (k < 0) return 0;
        kinds[i] = (uint8_t)k;
      }
      memcpy(counts, c->counts, 8);
      u128 r_arr = perm_rank(kinds, ORC_DIM, counts, c->n_kinds);
      local = (u128)gi * c->m_arr + r_arr;
    }
    *out = 1 + c->offset + (uint64_t)local;
    return 1;
  }
  return 0;
}

/* ======================================================================== */
/* FastDecoder — llvq-search/src/fastdec.rs                                   */
/* ======================================================================== */

/* fastdec.rs:173-194: M' = M c_j / n, exact at every step */
static void unrank_fast(uint64_t rank, uint8_t* counts, int k, uint64_t m0, uint8_t* out, int nslots) {
  uint64_t m = m0, n = (uint64_t)nslots;
  for (int s = 0; s < nslots; s++) {
    for (int j = 0; j < k; j++) {
      uint64_t c = counts[j];
      if (c == 0) continue;
      uint64_t mj = m * c / n;
      if (rank < mj) {
        out[s] = (uint8_t)j;
        counts[j]--;
        m = mj;
        break;
      }
      rank -= mj;
    }
    n--;
  }
}

int orc_class_of(uint64_t idx) { /* fastdec.rs:293-298 */
  ensure_init();
  if (idx == 0 || idx > ORC_N13) return -1;
  int lo = 0, hi = g_ncls;
  while (lo < hi) {
    int mid = (lo + hi) / 2;
    if (g_cls[mid].offset + g_cls[mid].card < idx) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

int orc_fast_decode(uint64_t idx, int32_t p[ORC_DIM]) { /* fastdec.rs:321-399 */
  ensure_init();
  memset(p, 0, sizeof(int32_t) * ORC_DIM);
  if (idx == 0) return 1;
  uint64_t i = idx - 1;
  if (i >= ORC_N13) return 0;
  const cls_t* c = &g_cls[find_class_linear(i)];
  uint64_t local = i - c->offset;
  if (c->odd) {
    uint64_t m_arr = (uint64_t)c->m_arr;
    uint64_t r_arr = local % m_arr;
    uint32_t cw = g_words[local / m_arr];
    uint8_t counts[8], kinds[ORC_DIM];
    memcpy(counts, c->counts, 8);
    unrank_fast(r_arr, counts, c->n_kinds, m_arr, kinds, ORC_DIM);
    for (int q = 0; q < ORC_DIM; q++) {
      int v = c->vals[kinds[q]];
      int a = (v % 4 == 3) ? v : -v;
      p[q] = ((cw >> q) & 1) ? a : -a;
    }
  } else {
    uint64_t s_f = (uint64_t)c->s_f, s_w = (uint64_t)c->s_w;
    uint64_t a_off = (uint64_t)c->a_off, a_on = (uint64_t)c->a_on;
    uint64_t r_sf = local % s_f; local /= s_f;
    uint64_t r_sw = local % s_w; local /= s_w;
    uint64_t r_off = local % a_off; local /= a_off;
    uint64_t r_on = local % a_on;
    uint32_t cw = g_words[g_start[c->w] + local / a_on];
    int w = c->w;
    uint8_t wc[8] = {0}, oc[8], on_kinds[ORC_DIM], off_kinds[ORC_DIM];
    memcpy(wc, c->word_counts, 4);
    memcpy(oc, c->off_counts, 8);
    unrank_fast(r_on, wc, c->n_word, a_on, on_kinds, w);
    unrank_fast(r_off, oc, c->n_off, a_off, off_kinds, ORC_DIM - w);
    uint32_t sign[ORC_DIM] = {0}, par = 0;
    for (int j = 0; j + 1 < w; j++) {
      sign[j] = (uint32_t)((r_sw >> j) & 1);
      par ^= sign[j];
    }
    if (w > 0) sign[w - 1] = par ^ (uint32_t)c->p_req;
    int zero_kind = c->n_off - 1, s_on = 0, s_off = 0, fbit = 0;
    for (int q = 0; q < ORC_DIM; q++) {
      if ((cw >> q) & 1) {
        int v = c->word_vals[on_kinds[s_on]];
        p[q] = sign[s_on] ? -v : v;
        s_on++;
      } else {
        int k = off_kinds[s_off];
        if (k != zero_kind) {
          int v = c->free_vals[k];
          p[q] = ((r_sf >> fbit) & 1) ? -v : v;
          fbit++;
        }
        s_off++;
      }
    }
  }
  return 1;
}

/* ======================================================================== */
/* Shell enumerators — llvq-core/src/shells.rs (test fixtures)                */
/* ======================================================================== */

typedef struct {
  int32_t* out;
  size_t cap, n;
  /* streaming check (orc_shell_roundtrip_check) */
  int check, shell, err;
  size_t stride;
  uint64_t lo, hi;
  uint8_t* seen;
} sink_t;

static void check_point(sink_t* s, const int32_t* x) {
  uint64_t idx;
  int32_t back[ORC_DIM];
  if (!orc_leech_contains(x) || orc_shell_index(x) != s->shell) { s->err = 1; return; }
  if (!orc_index_encode(x, &idx) || idx < s->lo || idx > s->hi) { s->err = 2; return; }
  if (s->seen[(idx - s->lo) >> 3] & (1u << ((idx - s->lo) & 7))) { s->err = 3; return; }
  s->seen[(idx - s->lo) >> 3] |= (uint8_t)(1u << ((idx - s->lo) & 7));
  if (!orc_index_decode(idx, back) || memcmp(back, x, sizeof back)) { s->err = 4; return; }
  if (!orc_fast_decode(idx, back) || memcmp(back, x, sizeof back)) { s->err = 5; return; }
}

static void emit(sink_t* s, const int32_t* x) {
  if (s->check) {
    if (!s->err && s->n % s->stride == 0) check_point(s, x);
  } else if (s->out && s->n < s->cap) {
    memcpy(s->out + s->n * ORC_DIM, x, sizeof(int32_t) * ORC_DIM);
  }
  s->n++;
}
static void ones_base(uint32_t c, int32_t* x) {
  for (int i = 0; i < ORC_DIM; i++) x[i] = ((c >> i) & 1) ? -1 : 1;
}
static void emit_two_support(sink_t* s, uint32_t support, int want_odd_minus, int extra_pos, int extra_val) {
  int pos[ORC_DIM], n = 0;
  for (int i = 0; i < ORC_DIM; i++)
    if ((support >> i) & 1) pos[n++] = i;
  for (uint32_t sg = 0; sg < (1u << n); sg++) {
    if ((popc(sg) & 1) != want_odd_minus) continue;
    int32_t x[ORC_DIM] = {0};
    for (int j = 0; j < n; j++) x[pos[j]] = ((sg >> j) & 1) ? -2 : 2;
    if (extra_pos >= 0) x[extra_pos] = extra_val;
    emit(s, x);
  }
}

static size_t enumerate_shell(int m, sink_t* sp);

size_t orc_enumerate_shell(int m, int32_t* out, size_t cap_points) {
  ensure_init();
  sink_t s;
  memset(&s, 0, sizeof s);
  s.out = out;
  s.cap = cap_points;
  return enumerate_shell(m, &s);
}

/* Every stride-th point of shell m (2 or 3) from the independent enumerator:
 * member of the lattice on shell m, encodes into [lo, hi] with no collision,
 * and both decoders return it.  Returns the number of points enumerated, or
 * the negated code of the first failure (1 membership, 2 range, 3 collision,
 * 4 Indexer round trip, 5 FastDecoder round trip). */
long long orc_shell_roundtrip_check(int m, size_t stride, uint64_t lo, uint64_t hi) {
  ensure_init();
  sink_t s;
  memset(&s, 0, sizeof s);
  s.check = 1;
  s.shell = m;
  s.stride = stride ? stride : 1;
  s.lo = lo;
  s.hi = hi;
  s.seen = (uint8_t*)calloc((size_t)((hi - lo) / 8 + 2), 1);
  size_t n = enumerate_shell(m, &s);
  free(s.seen);
  return s.err ? -(long long)s.err : (long long)n;
}

static size_t enumerate_shell(int m, sink_t* sp) {
  sink_t s = *sp;
  size_t ret = 0;
  if (m == 2) { /* shells.rs:66-92 */
    for (int i = g_start[8]; i < g_start[9]; i++) emit_two_support(&s, g_words[i], 0, -1, 0);
    for (int i = 0; i < ORC_DIM; i++)
      for (int j = i + 1; j < ORC_DIM; j++)
        for (int sg = 0; sg < 4; sg++) {
          int32_t x[ORC_DIM] = {0};
          x[i] = (sg & 1) ? -4 : 4;
          x[j] = (sg & 2) ? -4 : 4;
          emit(&s, x);
        }
    for (int g = 0; g < 4096; g++)
      for (int p = 0; p < ORC_DIM; p++) {
        int32_t x[ORC_DIM];
        ones_base(g_words[g], x);
        x[p] = ((g_words[g] >> p) & 1) ? 3 : -3;
        emit(&s, x);
      }
    ret = s.n;
    *sp = s;
    return ret;
  }
  if (m == 3) { /* shells.rs:94-143 */
    for (int i = g_start[12]; i < g_start[13]; i++) emit_two_support(&s, g_words[i], 0, -1, 0);
    for (int i = g_start[8]; i < g_start[9]; i++)
      for (int p4 = 0; p4 < ORC_DIM; p4++) {
        if ((g_words[i] >> p4) & 1) continue;
        emit_two_support(&s, g_words[i], 1, p4, 4);
        emit_two_support(&s, g_words[i], 1, p4, -4);
      }
    for (int g = 0; g < 4096; g++)
      for (int p = 0; p < ORC_DIM; p++) {
        int32_t x[ORC_DIM];
        ones_base(g_words[g], x);
        x[p] = ((g_words[g] >> p) & 1) ? -5 : 5;
        emit(&s, x);
      }
    for (int g = 0; g < 4096; g++)
      for (int i = 0; i < ORC_DIM; i++)
        for (int j = i + 1; j < ORC_DIM; j++)
          for (int k = j + 1; k < ORC_DIM; k++) {
            int32_t x[ORC_DIM];
            uint32_t c = g_words[g];
            ones_base(c, x);
            x[i] = ((c >> i) & 1) ? 3 : -3;
            x[j] = ((c >> j) & 1) ? 3 : -3;
            x[k] = ((c >> k) & 1) ? 3 : -3;
            emit(&s, x);
          }
    ret = s.n;
    *sp = s;
    return ret;
  }
  return 0;
}

/* ======================================================================== */
/* Bit stream — llvq-search/src/pack.rs                                       */
/* ======================================================================== */

struct orc_bitw {
  uint8_t* buf;
  size_t len, cap;
  uint64_t nbits; /* total bits pushed */
};
orc_bitw* orc_bitw_new(void) { return (orc_bitw*)calloc(1, sizeof(orc_bitw)); }
static void bitw_put(orc_bitw* w, int bit) {
  size_t byte = (size_t)(w->nbits >> 3);
  if (byte >= w->cap) {
    size_t nc = w->cap ? w->cap * 2 : 64;
    w->buf = (uint8_t*)realloc(w->buf, nc);
    memset(w->buf + w->cap, 0, nc - w->cap);
    w->cap = nc;
  }
  if (bit) w->buf[byte] |= (uint8_t)(0x80u >> (w->nbits & 7));
  w->nbits++;
  w->len = (size_t)((w->nbits + 7) >> 3);
}
int orc_bitw_push(orc_bitw* w, uint64_t value, uint32_t width) { /* pack.rs:48-82 */
  if (width > 64) return -1;
  if (width < 64 && value >= (1ULL << width)) return -1;
  for (uint32_t i = 0; i < width; i++) bitw_put(w, (int)((value >> (width - 1 - i)) & 1));
  return 0;
}
size_t orc_bitw_finish(orc_bitw* w, uint8_t** bytes) { /* pack.rs:90-98: final byte zero-padded */
  size_t n = w->len;
  *bytes = w->buf;
  if (!*bytes) *bytes = (uint8_t*)calloc(1, 1);
  free(w);
  return n;
}
uint64_t orc_bitr_read(const uint8_t* buf, uint64_t* pos, uint32_t width) { /* pack.rs:113-137 */
  uint64_t out = 0;
  for (uint32_t i = 0; i < width; i++) {
    uint64_t p = *pos + i;
    out = (out << 1) | ((buf[p >> 3] >> (7 - (p & 7))) & 1);
  }
  *pos += width;
  return out;
}
void orc_free(void* p) { free(p); }

/* ======================================================================== */
/* Fingerprint — llvq-artifact/src/codebook.rs:129-185                        */
/* ======================================================================== */

static uint64_t fnv_h;
static void fnv_byte(uint8_t b) {
  fnv_h ^= b;
  fnv_h *= 0x00000100000001b3ULL;
}
static void fnv_u64(uint64_t v) {
  for (int i = 0; i < 8; i++) fnv_byte((uint8_t)(v >> (8 * i)));
}
static void fnv_i32(int32_t v) {
  uint32_t u = (uint32_t)v;
  for (int i = 0; i < 4; i++) fnv_byte((uint8_t)(u >> (8 * i)));
}
static uint64_t fp_mix(uint64_t z) { /* codebook.rs:95-99 */
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
  return z ^ (z >> 31);
}
static void fp_probe(uint64_t idx) { /* codebook.rs:102-115 */
  int32_t p[ORC_DIM];
  fnv_u64(idx);
  if (orc_index_decode(idx, p)) {
    fnv_byte(1);
    for (int i = 0; i < ORC_DIM; i++) fnv_i32(p[i]);
  } else {
    fnv_byte(0);
  }
}
uint64_t orc_codebook_fingerprint(void) {
  ensure_init();
  static const char domain[] = "llvq codebook fingerprint v1";
  fnv_h = 0xcbf29ce484222325ULL;
  for (size_t i = 0; i + 1 < sizeof domain; i++) fnv_byte((uint8_t)domain[i]);
  fnv_u64(ORC_DIM);
  fnv_u64(ORC_N13);
  fnv_u64(GEN_POLY);
  fnv_u64(4096);
  for (int i = 0; i < 4096; i++) fnv_u64(g_words[i]);
  fnv_u64((uint64_t)g_ncls);
  for (int ci = 0; ci < g_ncls; ci++) {
    const cls_t* c = &g_cls[ci];
    uint64_t lo = c->offset + 1, hi = c->offset + c->card;
    fnv_u64(lo);
    fnv_u64(hi);
    fnv_u64((uint64_t)c->lv_len);
    fnv_u64((uint64_t)c->lv_nonzero);
    fnv_u64((uint64_t)c->odd);
    fnv_u64((uint64_t)c->shell);
    for (int k = 0; k < 5; k++) {
      fnv_i32(c->lv_values[k]);
      fnv_byte(c->lv_counts[k]);
    }
    uint64_t card = hi - lo + 1;
    for (uint64_t num = 0; num < 4; num++) fp_probe(lo + card * num / 4);
    fp_probe(hi);
    for (uint64_t k = 0; k < 2; k++) fp_probe(lo + fp_mix((uint64_t)ci ^ fp_mix(k)) % card);
  }
  fp_probe(0);
  fp_probe(ORC_N13 + 1);
  return fnv_h;
}

/* ======================================================================== */
/* Matrix record and header — llvq-artifact/src/format.rs                     */
/* ======================================================================== */

static int take(const uint8_t* buf, size_t len, size_t* pos, size_t n, const uint8_t** out) {
  if (n > len - *pos) return 0;
  *out = buf + *pos;
  *pos += n;
  return 1;
}
static int get_u32(const uint8_t* buf, size_t len, size_t* pos, uint32_t* v) {
  const uint8_t* p;
  if (!take(buf, len, pos, 4, &p)) return 0;
  *v = (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 | (uint32_t)p[3] << 24;
  return 1;
}
static int get_u64(const uint8_t* buf, size_t len, size_t* pos, uint64_t* v) {
  const uint8_t* p;
  if (!take(buf, len, pos, 8, &p)) return 0;
  uint64_t r = 0;
  for (int i = 7; i >= 0; i--) r = r << 8 | p[i];
  *v = r;
  return 1;
}
static void put_u32(uint8_t* p, uint32_t v) {
  for (int i = 0; i < 4; i++) p[i] = (uint8_t)(v >> (8 * i));
}
static void put_u64(uint8_t* p, uint64_t v) {
  for (int i = 0; i < 8; i++) p[i] = (uint8_t)(v >> (8 * i));
}

static int utf8_valid(const uint8_t* s, size_t n) {
  size_t i = 0;
  while (i < n) {
    uint8_t c = s[i];
    size_t need;
    uint32_t cp;
    if (c < 0x80) { i++; continue; }
    else if ((c & 0xE0) == 0xC0) { need = 1; cp = c & 0x1F; }
    else if ((c & 0xF0) == 0xE0) { need = 2; cp = c & 0x0F; }
    else if ((c & 0xF8) == 0xF0) { need = 3; cp = c & 0x07; }
    else return 0;
    for (size_t k = 1; k <= need; k++) {
      if (i + k >= n) return 0;
      if ((s[i + k] & 0xC0) != 0x80) return 0;
      cp = cp << 6 | (s[i + k] & 0x3F);
    }
    if ((need == 1 && cp < 0x80) || (need == 2 && cp < 0x800) || (need == 3 && cp < 0x10000)) return 0;
    if (cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return 0;
    i += need + 1;
  }
  return 1;
}

int orc_read_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                    uint32_t* n_matrices, const char** what) { /* format.rs:588-619 */
  const uint8_t* mg;
  const char* dummy;
  if (!what) what = &dummy;
  *what = "";
  if (!take(buf, len, pos, 4, &mg)) { *what = "magic"; return ORC_TRUNCATED; }
  if (!memcmp(mg, "LVQ4", 4)) *version = 4;
  else if (!memcmp(mg, "LVQ3", 4)) *version = 3;
  else if (!memcmp(mg, "LVQ2", 4)) *version = 2;
  else if (!memcmp(mg, "LVQ1", 4)) *version = 1;
  else return ORC_NOT_AN_ARTIFACT;
  if (!get_u32(buf, len, pos, n_matrices)) { *what = "matrix count"; return ORC_TRUNCATED; }
  if (*version >= 4) {
    uint64_t stored;
    if (!get_u64(buf, len, pos, &stored)) { *what = "codebook fingerprint"; return ORC_TRUNCATED; }
    if (stored != orc_codebook_fingerprint()) return ORC_CODEBOOK_MISMATCH;
  }
  return ORC_OK;
}

size_t orc_write_header(uint8_t* out, uint32_t version, uint32_t n_matrices) { /* format.rs:563-578 */
  static const char* magic[5] = {0, "LVQ1", "LVQ2", "LVQ3", "LVQ4"};
  if (version < 1 || version > 4) return 0;
  memcpy(out, magic[version], 4);
  put_u32(out + 4, n_matrices);
  if (version >= 4) {
    put_u64(out + 8, orc_codebook_fingerprint());
    return 16;
  }
  return 8;
}

static uint32_t gain_bits_of(uint32_t n_cent) { /* format.rs:87-89 */
  uint64_t p = 1;
  uint32_t b = 0;
  while (p < n_cent) { p <<= 1; b++; }
  return b;
}

void orc_raw_matrix_free(orc_raw_matrix* m) {
  free(m->name);
  free(m->centroids);
  free(m->row_scales);
  free(m->tail);
  free(m->indices);
  free(m->gains);
  memset(m, 0, sizeof *m);
}

int orc_read_matrix_raw(const uint8_t* buf, size_t len, size_t* pos, orc_raw_matrix* m,
                        const char** what) { /* format.rs:301-382 */
  ensure_init();
  const char* dummy;
  if (!what) what = &dummy;
  *what = "";
  memset(m, 0, sizeof *m);
  uint32_t nlen;
  const uint8_t* p;
#define FAIL(code, w) do { *what = (w); orc_raw_matrix_free(m); return (code); } while (0)
  if (!get_u32(buf, len, pos, &nlen)) FAIL(ORC_TRUNCATED, "name length");
  if (!take(buf, len, pos, nlen, &p)) FAIL(ORC_TRUNCATED, "name");
  if (!utf8_valid(p, nlen)) FAIL(ORC_BAD_NAME, "");
  m->name = (char*)malloc((size_t)nlen + 1);
  memcpy(m->name, p, nlen);
  m->name[nlen] = 0;
  if (!get_u32(buf, len, pos, &m->d_out)) FAIL(ORC_TRUNCATED, "d_out");
  if (!get_u32(buf, len, pos, &m->d_in)) FAIL(ORC_TRUNCATED, "d_in");
  if (!get_u32(buf, len, pos, &m->shell_cap)) FAIL(ORC_TRUNCATED, "shell cap");
  if (m->shell_cap > MAX_SHELL) FAIL(ORC_INCONSISTENT, "shell cap exceeds the supported ball");
  if (!get_u32(buf, len, pos, &m->n_centroids)) FAIL(ORC_TRUNCATED, "centroid count");
  if (!get_u64(buf, len, pos, &m->rot_seed)) FAIL(ORC_TRUNCATED, "rotation seed");
  uint32_t flag;
  if (!get_u32(buf, len, pos, &flag)) FAIL(ORC_TRUNCATED, "rotation flag");
  m->has_rot = flag != 0;

  if ((uint64_t)m->n_centroids * 8 > len - *pos) FAIL(ORC_TRUNCATED, "centroids");
  m->centroids = (double*)malloc(sizeof(double) * (m->n_centroids ? m->n_centroids : 1));
  for (uint32_t i = 0; i < m->n_centroids; i++) {
    uint64_t b;
    get_u64(buf, len, pos, &b);
    memcpy(&m->centroids[i], &b, 8);
  }
  if ((uint64_t)m->d_out * 8 > len - *pos) FAIL(ORC_TRUNCATED, "row scales");
  m->row_scales = (double*)malloc(sizeof(double) * (m->d_out ? m->d_out : 1));
  for (uint32_t i = 0; i < m->d_out; i++) {
    uint64_t b;
    get_u64(buf, len, pos, &b);
    memcpy(&m->row_scales[i], &b, 8);
  }
  uint64_t tail_n = (uint64_t)m->d_out * (m->d_in % ORC_DIM);
  if (tail_n * 4 > len - *pos) FAIL(ORC_TRUNCATED, "tail");
  m->tail = (double*)malloc(sizeof(double) * (tail_n ? tail_n : 1));
  for (uint64_t i = 0; i < tail_n; i++) {
    uint32_t b = 0;
    float f;
    get_u32(buf, len, pos, &b);
    memcpy(&f, &b, 4);
    m->tail[i] = (double)f;
  }
  uint64_t nbytes;
  if (!get_u64(buf, len, pos, &nbytes)) FAIL(ORC_TRUNCATED, "code length");
  if (nbytes > len - *pos) FAIL(ORC_TRUNCATED, "code stream");
  m->code_off = *pos;
  m->code_len = (size_t)nbytes;
  const uint8_t* codes = buf + *pos;
  *pos += (size_t)nbytes;

  uint32_t ib = (uint32_t)orc_index_bits(m->shell_cap), gb = gain_bits_of(m->n_centroids);
  uint64_t nblocks = (uint64_t)m->d_out * (m->d_in / ORC_DIM);
  u128 need = (u128)nblocks * (ib + gb);
  if (need > (u128)nbytes * 8) FAIL(ORC_TRUNCATED, "code stream");
  m->nblocks_total = (size_t)nblocks;
  m->indices = (uint64_t*)malloc(sizeof(uint64_t) * (nblocks ? nblocks : 1));
  m->gains = (uint32_t*)malloc(sizeof(uint32_t) * (nblocks ? nblocks : 1));
  uint64_t bp = 0;
  for (uint64_t b = 0; b < nblocks; b++) {
    m->indices[b] = orc_bitr_read(codes, &bp, ib);
    m->gains[b] = (uint32_t)orc_bitr_read(codes, &bp, gb);
  }
#undef FAIL
  return ORC_OK;
}

int orc_write_matrix_raw(const orc_raw_matrix* m, uint8_t** out, size_t* out_len) { /* format.rs:238-298 */
  ensure_init();
  size_t nb = (size_t)m->d_out * (m->d_in / ORC_DIM);
  if (m->nblocks_total != nb) return ORC_INCONSISTENT;
  uint32_t ib = (uint32_t)orc_index_bits(m->shell_cap), gb = gain_bits_of(m->n_centroids);
  orc_bitw* bw = orc_bitw_new();
  for (size_t b = 0; b < nb; b++) {
    if (ib < 64 && m->indices[b] >= (1ULL << ib)) {
      uint8_t* junk;
      orc_bitw_finish(bw, &junk);
      free(junk);
      return ORC_INDEX_TOO_WIDE;
    }
    if (orc_bitw_push(bw, m->indices[b], ib) || orc_bitw_push(bw, m->gains[b], gb)) {
      uint8_t* junk;
      orc_bitw_finish(bw, &junk);
      free(junk);
      return ORC_INCONSISTENT;
    }
  }
  uint8_t* codes;
  size_t clen = orc_bitw_finish(bw, &codes);
  size_t nlen = strlen(m->name);
  size_t tail_n = (size_t)m->d_out * (m->d_in % ORC_DIM);
  size_t total = 4 + nlen + 4 * 4 + 8 + 4 + 8 * (size_t)m->n_centroids + 8 * (size_t)m->d_out +
                 4 * tail_n + 8 + clen;
  uint8_t* o = (uint8_t*)malloc(total ? total : 1);
  size_t q = 0;
  put_u32(o + q, (uint32_t)nlen); q += 4;
  memcpy(o + q, m->name, nlen); q += nlen;
  put_u32(o + q, m->d_out); q += 4;
  put_u32(o + q, m->d_in); q += 4;
  put_u32(o + q, m->shell_cap); q += 4;
  put_u32(o + q, m->n_centroids); q += 4;
  put_u64(o + q, m->has_rot ? m->rot_seed : 0); q += 8;
  put_u32(o + q, m->has_rot ? 1 : 0); q += 4;
  for (uint32_t i = 0; i < m->n_centroids; i++) { uint64_t b; memcpy(&b, &m->centroids[i], 8); put_u64(o + q, b); q += 8; }
  for (uint32_t i = 0; i < m->d_out; i++) { uint64_t b; memcpy(&b, &m->row_scales[i], 8); put_u64(o + q, b); q += 8; }
  for (size_t i = 0; i < tail_n; i++) { float f = (float)m->tail[i]; uint32_t b; memcpy(&b, &f, 4); put_u32(o + q, b); q += 4; }
  put_u64(o + q, clen); q += 8;
  memcpy(o + q, codes, clen); q += clen;
  free(codes);
  *out = o;
  *out_len = q;
  return ORC_OK;
}

/* ======================================================================== */
/* reconstruct / decode_matrix / products                                     */
/* ======================================================================== */

void orc_reconstruct(const int32_t p[ORC_DIM], uint32_t gain, const double* centroids,
                     double row_scale, double out[ORC_DIM]) { /* quantizer.rs:354-367 */
  int64_t m = orc_shell_index(p);
  if (m > 0) {
    double picked = centroids[gain] * row_scale;
    double scale = picked / sqrt((double)(16 * m));
    for (int i = 0; i < ORC_DIM; i++) out[i] = (double)p[i] * scale;
  } else {
    for (int i = 0; i < ORC_DIM; i++) out[i] = 0.0;
  }
}

/* ---- rotation (llvq-quant/src/rotation.rs) ----------------------------- */
int orc_rotation_new(size_t n, uint64_t seed, orc_rotation* r) { /* rotation.rs:60-79 */
  memset(r, 0, sizeof *r);
  if (n == 0) return ORC_INCONSISTENT;
  size_t m = 1;
  while ((n & m) == 0) m <<= 1; /* 1 << n.trailing_zeros() */
  size_t k = n / m;
  r->n = n;
  r->m = m;
  r->k = k;
  r->signs = (double*)malloc(n * sizeof(double));
  r->small = (double*)malloc(k * k * sizeof(double));
  if (!r->signs || !r->small) return ORC_INCONSISTENT;
  uint64_t st = seed;
  for (size_t i = 0; i < n; i++) r->signs[i] = orc_splitmix_gaussian(&st) < 0.0 ? -1.0 : 1.0;
  /* orthonormal(k, rng), rotation.rs:226-247: Gram-Schmidt on Gaussian rows */
  double* row = (double*)malloc(k * sizeof(double));
  for (size_t i = 0; i < k; i++) {
    for (size_t t = 0; t < k; t++) row[t] = orc_splitmix_gaussian(&st);
    for (size_t p = 0; p < i; p++) {
      const double* prev = r->small + p * k;
      double d = 0.0;
      for (size_t t = 0; t < k; t++) d += row[t] * prev[t];
      for (size_t t = 0; t < k; t++) row[t] -= d * prev[t];
    }
    double nrm = 0.0;
    for (size_t t = 0; t < k; t++) nrm += row[t] * row[t];
    nrm = sqrt(nrm);
    for (size_t t = 0; t < k; t++) r->small[i * k + t] = row[t] / nrm;
  }
  free(row);
  return ORC_OK;
}

void orc_rotation_free(orc_rotation* r) {
  free(r->signs);
  free(r->small);
  memset(r, 0, sizeof *r);
}

static void orc_wht(double* v, size_t n) { /* rotation.rs:201-222 */
  for (size_t len = 1; len < n; len <<= 1)
    for (size_t i = 0; i < n; i += len << 1)
      for (size_t j = i; j < i + len; j++) {
        double a = v[j], b = v[j + len];
        v[j] = a + b;
        v[j + len] = a - b;
      }
  double s = 1.0 / sqrt((double)n);
  for (size_t i = 0; i < n; i++) v[i] *= s;
}

static void orc_rot_mix(const orc_rotation* r, double* v, int transpose) { /* rotation.rs:119-143 */
  if (r->k == 1) return;
  double* col = (double*)malloc(r->k * sizeof(double));
  for (size_t j = 0; j < r->m; j++) {
    for (size_t g = 0; g < r->k; g++) col[g] = v[g * r->m + j];
    for (size_t g = 0; g < r->k; g++) {
      double acc = 0.0;
      for (size_t t = 0; t < r->k; t++)
        acc += (transpose ? r->small[t * r->k + g] : r->small[g * r->k + t]) * col[t];
      v[g * r->m + j] = acc;
    }
  }
  free(col);
}

void orc_rotation_apply(const orc_rotation* r, double* v) { /* rotation.rs:97-105 */
  for (size_t i = 0; i < r->n; i++) v[i] *= r->signs[i];
  for (size_t g = 0; g < r->k; g++) orc_wht(v + g * r->m, r->m);
  orc_rot_mix(r, v, 0);
}

void orc_rotation_apply_transpose(const orc_rotation* r, double* v) { /* rotation.rs:108-117 */
  orc_rot_mix(r, v, 1);
  for (size_t g = 0; g < r->k; g++) orc_wht(v + g * r->m, r->m);
  for (size_t i = 0; i < r->n; i++) v[i] *= r->signs[i];
}

int orc_decode_matrix(const orc_raw_matrix* m, float* w) { /* format.rs:416-439 */
  size_t nb = m->d_in / ORC_DIM, tw = m->d_in % ORC_DIM;
  orc_rotation rot;
  memset(&rot, 0, sizeof rot);
  if (m->has_rot && orc_rotation_new(m->d_in, m->rot_seed, &rot) != ORC_OK) return ORC_INCONSISTENT;
  double* row = (double*)malloc(m->d_in * sizeof(double));
  int rc = ORC_OK;
  for (size_t r = 0; r < m->d_out && rc == ORC_OK; r++) {
    for (size_t b = 0; b < nb; b++) {
      int32_t p[ORC_DIM];
      size_t k = r * nb + b;
      if (!orc_index_decode(m->indices[k], p)) { rc = ORC_INDEX_OUT_OF_RANGE; break; }
      if (m->gains[k] >= m->n_centroids) { rc = ORC_INCONSISTENT; break; }
      orc_reconstruct(p, m->gains[k], m->centroids, m->row_scales[r], row + b * ORC_DIM);
    }
    if (rc != ORC_OK) break;
    for (size_t t = 0; t < tw; t++) row[nb * ORC_DIM + t] = m->tail[r * tw + t];
    if (m->has_rot) orc_rotation_apply_transpose(&rot, row); /* un-rotate in f64, then narrow */
    for (size_t c = 0; c < m->d_in; c++) w[r * m->d_in + c] = (float)row[c];
  }
  free(row);
  if (m->has_rot) orc_rotation_free(&rot);
  return rc;
}

int orc_fused_product(const orc_raw_matrix* m, const double* x_in, double* y, double* abs_out) {
  size_t nb = m->d_in / ORC_DIM, tw = m->d_in % ORC_DIM;
  double* xr = (double*)malloc(m->d_in * sizeof(double));
  memcpy(xr, x_in, m->d_in * sizeof(double));
  if (m->has_rot) { /* fused_path_matches_dense.rs:110-115: apply, not apply_transpose */
    orc_rotation rot;
    if (orc_rotation_new(m->d_in, m->rot_seed, &rot) != ORC_OK) { free(xr); return ORC_INCONSISTENT; }
    orc_rotation_apply(&rot, xr);
    orc_rotation_free(&rot);
  }
  const double* x = xr;
  int rc = ORC_OK;
  for (size_t r = 0; r < m->d_out && rc == ORC_OK; r++) {
    double acc = 0.0, aabs = 0.0;
    for (size_t b = 0; b < nb; b++) {
      int32_t p[ORC_DIM];
      size_t k = r * nb + b;
      if (!orc_fast_decode(m->indices[k], p)) { rc = ORC_INDEX_OUT_OF_RANGE; break; }
      if (m->gains[k] >= m->n_centroids) { rc = ORC_INCONSISTENT; break; }
      int64_t sh = orc_shell_index(p);
      if (sh > 0) {
        double kk = m->centroids[m->gains[k]] * m->row_scales[r] / sqrt((double)(16 * sh));
        for (int j = 0; j < ORC_DIM; j++) {
          double t = (double)p[j] * kk * x[b * ORC_DIM + j];
          acc += t;
          aabs += fabs(t);
        }
      }
    }
    for (size_t t = 0; t < tw; t++) {
      double v = m->tail[r * tw + t] * x[nb * ORC_DIM + t];
      acc += v;
      aabs += fabs(v);
    }
    y[r] = acc;
    if (abs_out) abs_out[r] = aabs;
  }
  free(xr);
  return rc;
}

void orc_dense_matvec(const float* w, size_t d_out, size_t d_in, const double* x, double* y) {
  for (size_t r = 0; r < d_out; r++) {
    double acc = 0.0;
    for (size_t c = 0; c < d_in; c++) acc += (double)w[r * d_in + c] * x[c];
    y[r] = acc;
  }
}

/* ======================================================================== */
/* f16 conversions                                                            */
/* ======================================================================== */

float orc_f16_to_f32(uint16_t h) { /* llvq-artifact/src/sealed.rs:47-62 */
  uint32_t sign = (uint32_t)(h >> 15) << 31;
  uint32_t e = (h >> 10) & 0x1F, f = h & 0x3FF, bits;
  if (e == 0) {
    if (f == 0) bits = sign;
    else {
      int sh = 0;
      while (!(f & 0x400)) { f <<= 1; sh++; }
      f &= 0x3FF;
      bits = sign | (uint32_t)(127 - 15 - sh + 1) << 23 | f << 13;
    }
  } else if (e == 31) {
    bits = sign | 0x7F800000u | f << 13;
  } else {
    bits = sign | (e + 127 - 15) << 23 | f << 13;
  }
  float r;
  memcpy(&r, &bits, 4);
  return r;
}

uint16_t orc_f32_to_f16(float fl) { /* llvq-cuda/src/lib.rs:60-96 — RNE */
  uint32_t x;
  memcpy(&x, &fl, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000);
  uint32_t e = (x >> 23) & 0xFF, f = x & 0x7FFFFF;
  if (e == 255) return (uint16_t)(sign | 0x7C00 | (f ? 0x200 | (f >> 13) : 0));
  int32_t ee = (int32_t)e - 127 + 15;
  if (ee >= 31) return (uint16_t)(sign | 0x7C00);
  if (ee <= 0) {
    if (ee < -10) return sign;
    f |= 0x800000;
    uint32_t shift = (uint32_t)(14 - ee);
    uint32_t half = f >> shift, rem = f & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1))) half++;
    return (uint16_t)(sign | half);
  }
  uint32_t half = (uint32_t)ee << 10 | f >> 13, rem = f & 0x1FFF;
  if (rem > 0x1000 || (rem == 0x1000 && (half & 1))) half++;
  return (uint16_t)(sign | half);
}

/* ======================================================================== */
/* Timed CPU baseline                                                          */
/* ======================================================================== */

static inline uint64_t be48(const uint8_t* p) {
  return (uint64_t)p[0] << 40 | (uint64_t)p[1] << 32 | (uint64_t)p[2] << 24 |
         (uint64_t)p[3] << 16 | (uint64_t)p[4] << 8 | (uint64_t)p[5];
}

typedef struct {
  const uint8_t* codes;
  size_t d_in, r0, r1;
  const double *centroids, *row_scales;
  const float* tail;
  const float* xf;
  float* y;
  int err;
} gemv_job;

static void* gemv_worker(void* arg) {
  gemv_job* j = (gemv_job*)arg;
  size_t nb = j->d_in / ORC_DIM, tw = j->d_in % ORC_DIM;
  for (size_t r = j->r0; r < j->r1; r++) {
    float acc = 0.f;
    for (size_t b = 0; b < nb; b++) {
      uint64_t v = be48(j->codes + 6 * (r * nb + b));
      int32_t p[ORC_DIM];
      double blk[ORC_DIM];
      if (!orc_fast_decode(v >> 1, p)) { j->err = ORC_INDEX_OUT_OF_RANGE; return 0; }
      orc_reconstruct(p, (uint32_t)(v & 1), j->centroids, j->row_scales[r], blk);
      const float* xb = j->xf + b * ORC_DIM;
      for (int q = 0; q < ORC_DIM; q++) acc += (float)blk[q] * xb[q];
    }
    for (size_t t = 0; t < tw; t++) acc += j->tail[r * tw + t] * j->xf[nb * ORC_DIM + t];
    j->y[r] = acc;
  }
  return 0;
}

int orc_cpu_gemv(const uint8_t* codes, size_t d_out, size_t d_in, const double* centroids,
                 const double* row_scales, const float* tail, const uint16_t* x_f16, float* y,
                 int threads) {
  ensure_init();
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  float* xf = (float*)malloc(sizeof(float) * (d_in ? d_in : 1));
  for (size_t i = 0; i < d_in; i++) xf[i] = orc_f16_to_f32(x_f16[i]);
  pthread_t th[256];
  gemv_job jobs[256];
  size_t per = (d_out + (size_t)threads - 1) / (size_t)threads;
  int started = 0;
  for (int t = 0; t < threads; t++) {
    size_t r0 = (size_t)t * per, r1 = r0 + per > d_out ? d_out : r0 + per;
    if (r0 >= r1) break;
    jobs[t] = (gemv_job){codes, d_in, r0, r1, centroids, row_scales, tail, xf, y, 0};
    pthread_create(&th[t], 0, gemv_worker, &jobs[t]);
    started++;
  }
  int err = 0;
  for (int t = 0; t < started; t++) {
    pthread_join(th[t], 0);
    if (jobs[t].err) err = jobs[t].err;
  }
  free(xf);
  return err;
}

int orc_decode_batch(const uint64_t* idx, size_t n, int8_t* out, int fast) {
  ensure_init();
  for (size_t k = 0; k < n; k++) {
    int32_t p[ORC_DIM];
    int ok = fast ? orc_fast_decode(idx[k], p) : orc_index_decode(idx[k], p);
    if (!ok) return ORC_INDEX_OUT_OF_RANGE;
    for (int q = 0; q < ORC_DIM; q++) out[k * ORC_DIM + q] = (int8_t)p[q];
  }
  return ORC_OK;
}

uint64_t orc_cpu_decode_only(const uint8_t* codes, size_t nblocks) {
  ensure_init();
  uint64_t sum = 0;
  for (size_t b = 0; b < nblocks; b++) {
    int32_t p[ORC_DIM];
    uint64_t v = be48(codes + 6 * b);
    orc_fast_decode(v >> 1, p);
    for (int q = 0; q < ORC_DIM; q++) sum = sum * 31 + (uint64_t)(uint32_t)p[q];
  }
  return sum;
}
