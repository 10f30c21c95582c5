/* pool_planner_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A plain-C restatement of the reference's memory-pool address simulator
 * (src/Transform/DNN/mallocPoolOpt.hpp in the reference tree), written from
 * that header's semantics function by function.  The header itself cannot be
 * compiled here (it needs MLIR), so this restatement is pinned by the two
 * worked traces recorded from the reference planner core (tests/golden/
 * planner_*.json) and, for what those leave open, by an independent granule
 * bitmap model and interval invariants (tests/test_planner.py).
 *
 * Blocks carry INCLUSIVE end addresses, as in the reference
 * (mallocPoolOpt.hpp:7-16), and the free list starts as one block
 * [0, INT64_MAX-1] (:18).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct { int64_t start, end; } FreeBlk;
typedef struct { int64_t id, start, end; } AllocBlk;

typedef struct {
  FreeBlk *fr; int nfr, cfr;
  AllocBlk *al; int nal, cal;
  int64_t peak;
} Sim;

static void fr_insert(Sim *s, int at, FreeBlk b) {
  if (s->nfr == s->cfr) { s->cfr = s->cfr ? 2 * s->cfr : 16; s->fr = realloc(s->fr, sizeof(FreeBlk) * s->cfr); }
  memmove(s->fr + at + 1, s->fr + at, sizeof(FreeBlk) * (s->nfr - at));
  s->fr[at] = b; s->nfr++;
}
static void fr_erase(Sim *s, int at) {
  memmove(s->fr + at, s->fr + at + 1, sizeof(FreeBlk) * (s->nfr - at - 1));
  s->nfr--;
}
static void al_insert(Sim *s, int at, AllocBlk b) {
  if (s->nal == s->cal) { s->cal = s->cal ? 2 * s->cal : 16; s->al = realloc(s->al, sizeof(AllocBlk) * s->cal); }
  memmove(s->al + at + 1, s->al + at, sizeof(AllocBlk) * (s->nal - at));
  s->al[at] = b; s->nal++;
}
static void al_erase(Sim *s, int at) {
  memmove(s->al + at, s->al + at + 1, sizeof(AllocBlk) * (s->nal - at - 1));
  s->nal--;
}

/* mallocPoolOpt.hpp:21-37 getMemRefSize: bytes rounded up to a multiple of 32,
 * non-positive sizes become 0. */
int64_t oracle_round_size(int64_t bytes) {
  return bytes <= 0 ? 0 : ((bytes - 1) / 32 + 1) * 32;
}

/* mallocPoolOpt.hpp:46-53 findFirstFit: the first block whose end - start
 * is >= size.  Ends are inclusive, so a block of exactly `size` bytes has
 * end - start == size - 1 and does NOT fit. */
static int find_first_fit(const Sim *s, int64_t size) {
  for (int i = 0; i < s->nfr; i++)
    if (s->fr[i].end - s->fr[i].start >= size) return i;
  return -1;
}

/* mallocPoolOpt.hpp:69-96 mallocSimul: carve [start, start+size-1] off the
 * front of the chosen block; keep the alloc list sorted by start, inserting
 * before the first entry whose start is not below the new start. */
static int64_t malloc_simul(Sim *s, int64_t id, int64_t size) {
  const int fi = find_first_fit(s, size);
  if (fi < 0) return -1;
  const FreeBlk fb = s->fr[fi];
  const AllocBlk ab = {id, fb.start, fb.start + size - 1};
  if (s->nal == 0) {
    al_insert(s, 0, ab);
    s->fr[fi].start += size;
    return ab.start;
  }
  for (int ai = 0; ai < s->nal; ai++) {
    if (s->al[ai].start < fb.start) {
      if (ai == s->nal - 1) {
        al_insert(s, s->nal, ab);
        s->fr[fi].start += size;
        return ab.start;
      }
      continue;
    }
    al_insert(s, ai, ab);
    s->fr[fi].start += size;
    return ab.start;
  }
  return -1;
}

/* mallocPoolOpt.hpp:98-140 deallocSimul. */
static int dealloc_simul(Sim *s, int64_t id) {
  for (int ai = 0; ai < s->nal; ai++) {
    if (s->al[ai].id != id) continue;
    const AllocBlk d = s->al[ai];
    al_erase(s, ai);
    for (int fi = 0; fi < s->nfr; fi++) {
      if (s->fr[fi].end == d.start - 1) { /* free block right below */
        s->fr[fi].end = d.end;
        if (fi < s->nfr - 1 && s->fr[fi + 1].start == s->fr[fi].end + 1) {
          s->fr[fi + 1].start = s->fr[fi].start;
          fr_erase(s, fi);
        }
        return 1;
      } else if (s->fr[fi].start == d.end + 1) { /* free block right above */
        s->fr[fi].start = d.start;
        if (fi > 0 && s->fr[fi - 1].end == s->fr[fi].start - 1) {
          s->fr[fi - 1].end = s->fr[fi].end;
          fr_erase(s, fi);
        }
        return 1;
      }
    }
    for (int fi = 0; fi < s->nfr; fi++) { /* no neighbour: insert in order */
      const FreeBlk nf = {d.start, d.end};
      if (s->fr[fi].start > d.end) { fr_insert(s, fi, nf); return 1; }
      else if (fi == s->nfr - 1 && s->fr[fi].start < d.end) { fr_insert(s, s->nfr, nf); return 1; }
    }
    /* the reference's outer loop goes on to the next alloc entry here */
  }
  return 0;
}

/* Replays a trace.  kind[i] 0 = malloc of bytes[i] (already a raw byte count;
 * rounding is applied here), 1 = dealloc; id[i] names the tensor.  Writes the
 * offset of every malloc event to offset[i] (-1 for dealloc events) and
 * returns the pool size: the running maximum, taken after every event, of the
 * start of the last free block (mallocPoolOpt.hpp:212-218, driver loop
 * mallocPoolOpt.cpp:41-76).  Returns -1 if a dealloc names no live tensor. */
int64_t oracle_plan_pool(int64_t n, const int32_t *kind, const int64_t *id,
                         const int64_t *bytes, int64_t *offset) {
  Sim s; memset(&s, 0, sizeof s);
  const FreeBlk init = {0, INT64_MAX - 1};
  fr_insert(&s, 0, init);
  int64_t ret = 0;
  for (int64_t i = 0; i < n; i++) {
    if (kind[i] == 0) {
      offset[i] = malloc_simul(&s, id[i], oracle_round_size(bytes[i]));
      if (offset[i] < 0) { ret = -1; break; }
    } else {
      offset[i] = -1;
      if (!dealloc_simul(&s, id[i])) { ret = -1; break; }
    }
    if (s.peak < s.fr[s.nfr - 1].start) s.peak = s.fr[s.nfr - 1].start;
  }
  if (ret == 0) ret = s.peak;
  free(s.fr); free(s.al);
  return ret;
}

/* Same replay, also dumping the free list after event `upto` (for the golden
 * traces, which record it after each dealloc).  out holds 2*cap int64. */
int64_t oracle_free_list_after(int64_t n, const int32_t *kind, const int64_t *id,
                               const int64_t *bytes, int64_t upto, int64_t *out,
                               int64_t cap) {
  Sim s; memset(&s, 0, sizeof s);
  const FreeBlk init = {0, INT64_MAX - 1};
  fr_insert(&s, 0, init);
  for (int64_t i = 0; i <= upto && i < n; i++) {
    if (kind[i] == 0) malloc_simul(&s, id[i], oracle_round_size(bytes[i]));
    else dealloc_simul(&s, id[i]);
  }
  int64_t m = s.nfr;
  for (int64_t i = 0; i < m && i < cap; i++) { out[2 * i] = s.fr[i].start; out[2 * i + 1] = s.fr[i].end; }
  free(s.fr); free(s.al);
  return m;
}
