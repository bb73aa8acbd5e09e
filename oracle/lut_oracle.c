/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of the look-up-table algorithms of
 * ptillet/torch-blocksparse.  Nothing in the shipped library links, loads or calls this file; only
 * the tests, the smoke check and the CPU-baseline leg of the benchmark may use it, as the checker.
 *
 * Every function cites the reference lines it follows.  The restatement is sequential and literal on
 * purpose (the product builds the same tables with parallel device kernels, so the two are independent
 * derivations of the same tables).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_sdd_segment        : against the reference's own C++ (csrc/utils.cpp compiled into oracle/_ref)
 *                            on random layouts + committed golden fixtures + closed form at width 1.
 *   orc_make_layout_cpp    : against oracle/_ref make_layout + committed golden fixtures.
 *   orc_make_layout_py     : golden layouts written by the reference's own _make_layout (vertical stripes of 1-4 blocks).
 *   orc_softmax_lut        : closed form from nonzero()/cumsum + hand-derived known answer.
 *   orc_load_balance,
 *   orc_dxx_lut            : committed golden fixtures generated from the reference's Python
 *                            (tests/golden/make_golden.py), the hand-derived known answer, and the
 *                            structural invariants (walking the increments visits every block once).
 *
 * All tables use int64 arithmetic and are truncated to int32 at the end, like the reference
 * (`lut.type(torch.int32)`, matmul.py:455, softmax.py:220).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR_ALLOC (-1)
#define ORC_ERR_EMPTY_HEAD (-2) /* reference raises: min()/max() of an empty tensor, division by 0 */
#define ORC_ERR_CAPACITY (-3)

static int64_t at3(const int32_t *a, int R, int C, int h, int r, int c) { return a[((int64_t)h * R + r) * C + c]; }

/* ------------------------------------------------------------------------------------------------
 * sdd look-up table.  Reference: csrc/utils.cpp:11-120 (segment_blocks, sdd_segment) and
 * matmul.py:281-297 (make_sdd_lut flattens each table to int32 [n*4], width = rows/(w*w)).
 *
 * layout : int32 [H,R,C], consumed (retained entries are zeroed, utils.cpp:75).
 * out    : int32 [nnz*4] rows (h, i, j, blockid), all pack levels back to back in the order the
 *          reference returns them (start_width first).
 * packs/rows : per emitted level, its pack size and its number of rows; *n_levels levels.
 * ------------------------------------------------------------------------------------------------ */
static int segment_level(int32_t *layout, const int32_t *rank, int H, int R, int C, int w,
                         int32_t *tmp, int32_t *out, int64_t out_cap, int64_t *out_rows) {
  /* utils.cpp:15 tmp = zeros_like(layout) per level */
  memset(tmp, 0, sizeof(int32_t) * (size_t)H * R * C);
  int *left = (int *)malloc(sizeof(int) * (size_t)w);
  int *top = (int *)malloc(sizeof(int) * (size_t)w * C);
  if (!left || !top) { free(left); free(top); return ORC_ERR_ALLOC; }
  int64_t rows = 0;
  for (int h = 0; h < H; h++) { /* utils.cpp:28 (heads are independent; per-head output concatenated in head order, :86-91) */
    for (int k = 0; k < w; k++) left[k] = -1;           /* utils.cpp:31: declared per head, NOT reset per row */
    for (int k = 0; k < w * C; k++) top[k] = -1;        /* utils.cpp:32 */
    for (int m = 0; m < R; m++)
      for (int n = 0; n < C; n++) {
        if (layout[((int64_t)h * R + m) * C + n] == 0) continue;          /* :36-38 */
        int n_left = left[w - 1];                                          /* :39 */
        int m_top = top[(w - 1) * C + n];                                  /* :40 */
        int t = (m_top >= 0) ? tmp[((int64_t)h * R + m_top) * C + n] : 0;  /* :41 */
        int l = (n_left >= 0) ? tmp[((int64_t)h * R + m) * C + n_left] : 0; /* :42 */
        int tl = (m_top >= 0 && n_left >= 0) ? tmp[((int64_t)h * R + m_top) * C + n_left] : 0; /* :43 */
        int width = (l < t ? l : t);
        width = (width < tl ? width : tl) + 1;                             /* :44 */
        for (int nn = n_left + 1; nn < n; nn++)                            /* :48-50 */
          if (top[(w - 1) * C + nn] > top[(w - 1) * C + n]) width = 1;
        tmp[((int64_t)h * R + m) * C + n] = width;                         /* :51 */
        for (int k = 0; k < w - 1; k++) left[k] = left[k + 1];             /* :54-56 */
        left[w - 1] = n;
        for (int k = 0; k < w - 1; k++) top[k * C + n] = top[(k + 1) * C + n]; /* :59-61 */
        top[(w - 1) * C + n] = m;
        if (width != w) continue;                                          /* :64-65 */
        for (int km = 0; km < w; km++)
          for (int kn = 0; kn < w; kn++) {                                 /* :68-82 */
            int mm = top[km * C + n], nn = left[kn];
            if (mm < 0 || nn < 0) continue;
            int64_t p = ((int64_t)h * R + mm) * C + nn;
            layout[p] = 0;
            tmp[p] = 0;
            if (rows >= out_cap) { free(left); free(top); return ORC_ERR_CAPACITY; }
            out[rows * 4 + 0] = h; out[rows * 4 + 1] = mm; out[rows * 4 + 2] = nn; out[rows * 4 + 3] = rank[p];
            rows++;
          }
      }
  }
  free(left); free(top);
  *out_rows = rows;
  return ORC_OK;
}

int orc_sdd_segment(int32_t *layout, int H, int R, int C, int start_width, int32_t *out, int64_t out_cap_rows,
                    int32_t *packs, int64_t *rows, int *n_levels) {
  size_t n = (size_t)H * R * C;
  int32_t *rank = (int32_t *)calloc(n ? n : 1, sizeof(int32_t));
  int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * (n ? n : 1));
  if (!rank || !tmp) { free(rank); free(tmp); return ORC_ERR_ALLOC; }
  int32_t cur = 0; /* utils.cpp:99-112: running index of nonzeros in (h,m,n) order */
  for (size_t p = 0; p < n; p++) if (layout[p] != 0) rank[p] = cur++;
  int levels = 0; int64_t done = 0; int rc = ORC_OK;
  for (int w = start_width; w > 0; w /= 2) { /* utils.cpp:117-118 */
    int64_t r = 0;
    rc = segment_level(layout, rank, H, R, C, w, tmp, out + done * 4, out_cap_rows - done, &r);
    if (rc != ORC_OK) break;
    if (r > 0) { packs[levels] = w; rows[levels] = r; levels++; done += r; } /* :88-91: empty levels are not returned */
  }
  *n_levels = levels;
  free(rank); free(tmp);
  return rc;
}

/* ------------------------------------------------------------------------------------------------
 * load_balance.  Reference: matmul.py:221-267.  sizes[n] -> segments/column/lockid/maxid/offsets,
 * each of length *width (capacity cap).  `block` is unused by the reference too.
 * ------------------------------------------------------------------------------------------------ */
static int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

int orc_load_balance(const int64_t *sizes, int n, int64_t *segments, int64_t *column, int64_t *lockid,
                     int64_t *maxid, int64_t *offsets, int cap, int *width) {
  int64_t max_size = 0; int any = 0;
  for (int i = 0; i < n; i++) { if (sizes[i] > max_size) max_size = sizes[i]; if (sizes[i] != 0) any = 1; }
  if (!any || n == 0) return ORC_ERR_EMPTY_HEAD;            /* :226-227 raise on an all-zero head */
  int64_t seg_max = max_size;                                /* :232 */
  int64_t seg_min = cdiv64(seg_max, 4) > 4 ? cdiv64(seg_max, 4) : 4; /* :233 */
  int64_t total = 0;
  for (int i = 0; i < n; i++)                                /* :235-238 */
    total += sizes[i] / seg_max + (sizes[i] < seg_min) + (sizes[i] % seg_max >= seg_min);
  if (total > cap) return ORC_ERR_CAPACITY;
  for (int64_t s = 0; s < total; s++) { lockid[s] = 0; maxid[s] = 0; segments[s] = 0; column[s] = 0; }
  int64_t nlocks = 0, current = 0;
  for (int i = 0; i < n; i++) {                              /* :246-264 */
    int64_t d = sizes[i] / seg_max, r = sizes[i] % seg_max;
    int isempty = sizes[i] < seg_min;
    int64_t last = current + d + (r >= seg_min) + isempty;
    for (int64_t s = current; s < last; s++) column[s] = i;
    if (d > 1 || (d == 1 && r >= seg_min)) {
      nlocks++;
      for (int64_t s = current; s < last; s++) { lockid[s] = nlocks; maxid[s] = last - current; }
    }
    for (int64_t s = current; s < current + d; s++) segments[s] = seg_max;
    if (r < seg_min && !isempty) segments[current + d - 1] += r;
    if (r >= seg_min || isempty) segments[current + d] = r;
    current = last;
  }
  offsets[0] = 0;                                            /* :265-266 */
  for (int64_t s = 1; s < total; s++) offsets[s] = offsets[s - 1] + segments[s - 1];
  *width = (int)total;
  return ORC_OK;
}

/* ------------------------------------------------------------------------------------------------
 * dsd/dds look-up table.  Reference: matmul.py:372-458 (make_dxx_lut, identity `transform`).
 * layout int32 [H,R,C] (read-only).  lut capacity lut_cap int32; on success *lut_len ints written,
 * *width = number of segments, *num_locks as the reference returns it.
 * ------------------------------------------------------------------------------------------------ */
int orc_dxx_lut(const int32_t *layout, int H, int R, int C, int block, int step, int trans, int32_t *lut,
                int64_t lut_cap, int64_t *lut_len, int *width_out, int *num_locks_out) {
  int L = trans ? R : C;                /* number of reduction lines per head */
  int cap = 2 * H * L + 2;
  int64_t *seg = malloc(sizeof(int64_t) * cap), *col = malloc(sizeof(int64_t) * cap), *dep = malloc(sizeof(int64_t) * cap),
          *lck = malloc(sizeof(int64_t) * cap), *mxd = malloc(sizeof(int64_t) * cap), *off = malloc(sizeof(int64_t) * cap),
          *sizes = malloc(sizeof(int64_t) * (L ? L : 1));
  int64_t nnz_total = 0;
  for (int64_t p = 0; p < (int64_t)H * R * C; p++) nnz_total += layout[p] != 0;
  int64_t *idx = malloc(sizeof(int64_t) * (nnz_total ? nnz_total : 1)), *widx = malloc(sizeof(int64_t) * (nnz_total ? nnz_total : 1));
  int64_t ncell = (int64_t)H * R * C;
  int64_t *rank = malloc(sizeof(int64_t) * (ncell > 0 ? ncell : 1));
  int rc = ORC_OK;
  if (!seg || !col || !dep || !lck || !mxd || !off || !sizes || !idx || !widx || !rank) { rc = ORC_ERR_ALLOC; goto done; }
  {
    int width = 0; int64_t current_offset = 0, current_maxid = 0;
    for (int z = 0; z < H; z++) {        /* :384-400 */
      int64_t head_nnz = 0;
      for (int i = 0; i < L; i++) {
        int64_t s = 0;
        if (trans) for (int c = 0; c < C; c++) s += at3(layout, R, C, z, i, c);      /* :386 sum over dim 1 of [R,C] */
        else       for (int r = 0; r < R; r++) s += at3(layout, R, C, z, r, i);      /* :388 */
        sizes[i] = s; head_nnz += s;
      }
      int w = 0;
      rc = orc_load_balance(sizes, L, seg + width, col + width, lck + width, mxd + width, off + width, cap - width, &w);
      if (rc != ORC_OK) goto done;
      int64_t zmax = 0;
      for (int s = width; s < width + w; s++) {
        dep[s] = z;                                                  /* :390 */
        if (lck[s] > 0) lck[s] += current_maxid;                     /* :391 */
        if (lck[s] > zmax) zmax = lck[s];
        off[s] += current_offset;                                    /* :398 */
      }
      current_maxid = zmax;                                          /* :392 (max of this head only) */
      current_offset += head_nnz;                                    /* :400 */
      width += w;
    }
    for (int s = 0; s < width; s++) seg[s] *= step;                  /* :401 */
    int64_t num_blocks = nnz_total;                                  /* :407 */
    if (num_blocks == 0) { rc = ORC_ERR_EMPTY_HEAD; goto done; }
    for (int s = 0; s < width; s++) if (off[s] > num_blocks - 1) off[s] = num_blocks - 1; /* :408 */
    /* storage rank of every nonzero in (h,r,c) order */
    { int64_t cur = 0; for (int64_t p = 0; p < (int64_t)H * R * C; p++) rank[p] = layout[p] != 0 ? cur++ : -1; }
    /* :403-409 and :421-432: walk the nonzeros in (h,r,c) order (trans) or (h,c,r) order (not trans) */
    {
      int64_t t = 0;
      for (int z = 0; z < H; z++) {
        if (trans) {
          for (int r = 0; r < R; r++) for (int c = 0; c < C; c++)
            if (at3(layout, R, C, z, r, c)) { idx[t] = (int64_t)c * block; widx[t] = t; t++; }   /* nnz[:,2]*block ; arange */
        } else {
          for (int c = 0; c < C; c++) for (int r = 0; r < R; r++)
            if (at3(layout, R, C, z, r, c)) { idx[t] = (int64_t)r * block; widx[t] = rank[((int64_t)z * R + r) * C + c]; t++; }
        }
      }
    }
    int div = block / step;                                          /* :413 */
    if (div < 1) { rc = ORC_ERR_CAPACITY; goto done; }
    int64_t need = 6 * (int64_t)width + 2 * num_blocks * div + 2;
    if (need > lut_cap) { rc = ORC_ERR_CAPACITY; goto done; }
    int64_t *inc = malloc(sizeof(int64_t) * 2 * num_blocks * div);
    if (!inc) { rc = ORC_ERR_ALLOC; goto done; }
    int64_t wstep = trans ? step : (int64_t)step * block;            /* :436-441 */
    for (int64_t t = 0; t < num_blocks; t++) {
      int64_t dx = idx[t] - (t ? idx[t - 1] : 0);                    /* :410-411 */
      int64_t dw = widx[t] * block * block - (t ? widx[t - 1] * block * block : 0); /* :433-434 */
      for (int j = 0; j < div; j++) {
        inc[(t * div + j) * 2 + 0] = j ? step : dx - (int64_t)(div - 1) * step;      /* :414-416 */
        inc[(t * div + j) * 2 + 1] = j ? wstep : dw - (int64_t)(div - 1) * wstep;
      }
    }
    for (int s = 0; s < width; s++)                                  /* :418 and :442, segments > 0 only */
      if (seg[s] > 0) { inc[(off[s] * div) * 2 + 0] = idx[off[s]]; inc[(off[s] * div) * 2 + 1] = widx[off[s]]; }
    int64_t lockmax = 0;
    for (int s = 0; s < width; s++) {                                /* :445-450 */
      lut[s * 6 + 0] = (int32_t)(off[s] * 2 * div + 6 * (int64_t)width);
      lut[s * 6 + 1] = (int32_t)(seg[s] * div);
      lut[s * 6 + 2] = (int32_t)col[s];
      lut[s * 6 + 3] = (int32_t)dep[s];
      lut[s * 6 + 4] = (int32_t)lck[s];
      lut[s * 6 + 5] = (int32_t)mxd[s];
      if (lck[s] > lockmax) lockmax = lck[s];
    }
    for (int64_t q = 0; q < 2 * num_blocks * div; q++) lut[6 * (int64_t)width + q] = (int32_t)inc[q]; /* :451 */
    lut[need - 2] = 0; lut[need - 1] = 0;                             /* :452 */
    free(inc);
    *lut_len = need; *width_out = width; *num_locks_out = lockmax > 1 ? (int)lockmax : 1; /* :457 */
  }
done:
  free(seg); free(col); free(dep); free(lck); free(mxd); free(off); free(sizes); free(idx); free(widx); free(rank);
  return rc;
}

/* ------------------------------------------------------------------------------------------------
 * softmax look-up table.  Reference: softmax.py:201-221.  lut int32 [2*H*R + 4*nnz].
 * ------------------------------------------------------------------------------------------------ */
int orc_softmax_lut(const int32_t *layout, int H, int R, int C, int32_t *lut, int64_t lut_cap, int64_t *lut_len, int *maxlut) {
  int64_t nrows = (int64_t)H * R, nnz = 0, mx = 0;
  for (int64_t p = 0; p < nrows * C; p++) nnz += layout[p];   /* layout.sum(): values are 0/1 */
  if (2 * nrows + 4 * nnz > lut_cap) return ORC_ERR_CAPACITY;
  int64_t cum = 0, t = 0;
  for (int h = 0; h < H; h++) for (int r = 0; r < R; r++) {
    int64_t size = 0;
    for (int c = 0; c < C; c++) size += at3(layout, R, C, h, r, c);  /* :206-207 */
    lut[((int64_t)h * R + r) * 2 + 0] = (int32_t)size;
    lut[((int64_t)h * R + r) * 2 + 1] = (int32_t)(cum * 4 + 2 * nrows); /* :209-210, :218 */
    cum += size; if (size > mx) mx = size;
    for (int c = 0; c < C; c++) if (at3(layout, R, C, h, r, c)) {      /* :212-216 core = (idx, col, row, head) */
      int32_t *e = lut + 2 * nrows + 4 * t;
      e[0] = (int32_t)t; e[1] = c; e[2] = r; e[3] = h; t++;
    }
  }
  *lut_len = 2 * nrows + 4 * nnz; *maxlut = (int)mx;                   /* :221 */
  return ORC_OK;
}

/* ------------------------------------------------------------------------------------------------
 * Layout generators.  out int64 [H, nb, nb].
 *  orc_make_layout_cpp : csrc/utils.cpp:123-148 (exposed as torch_blocksparse.attention.make_layout)
 *  orc_make_layout_py  : deepspeedsparseselfattention.py:31-65 (_set_s1_layout/_set_s2_layout/_make_layout)
 * They differ for vertsize > 1 (utils.cpp:143 advances k by num_blocks, the Python clamps a range).
 * ------------------------------------------------------------------------------------------------ */
void orc_make_layout_cpp(int H, int nb, int dense, int stride, int unidirectional, int numverts, int vertsize, int64_t *out) {
  for (int64_t p = 0; p < (int64_t)H * nb * nb; p++) out[p] = dense ? 1 : 0;
  if (dense) return;
  for (int h = 0; h < H; h++) {
    int64_t *L = out + (int64_t)h * nb * nb;
    for (int i = 0; i < nb; i += stride)                      /* :133-136 (caller guarantees stride | nb, else the reference writes out of bounds) */
      for (int j = i; j < i + stride; j++)
        for (int k = i; k < (unidirectional ? j + 1 : i + stride); k++) L[(int64_t)j * nb + k] = 1;
    int start = stride - (1 + h % numverts) * vertsize;       /* :139 */
    for (int i = 0; i < nb; i++) {
      int end = unidirectional ? i : nb;                      /* :141 */
      for (int j = start; j < end; j += stride)
        for (int k = j; k < j + vertsize; k += nb) L[(int64_t)i * nb + k] = 1; /* :143-144 */
    }
  }
}

void orc_make_layout_py(int H, int nb, int dense, int stride, int unidirectional, int numverts, int vertsize, int64_t *out) {
  for (int64_t p = 0; p < (int64_t)H * nb * nb; p++) out[p] = dense ? 1 : 0;
  if (dense) return;
  for (int h = 0; h < H; h++) {
    int64_t *L = out + (int64_t)h * nb * nb;
    for (int i = 0; i < nb; i += stride)                      /* _set_s1_layout :33-37 */
      for (int j = i; j < i + stride; j++)
        for (int k = i; k < (unidirectional ? j + 1 : i + stride); k++) L[(int64_t)j * nb + k] = 1;
    int start = stride - (1 + h % numverts) * vertsize;       /* _set_s2_layout :41-47 */
    for (int i = 0; i < nb; i++) {
      int end = unidirectional ? i : nb;
      for (int j = start; j < end; j += stride)
        for (int k = j; k < (j + vertsize < nb ? j + vertsize : nb); k++) L[(int64_t)i * nb + k] = 1;
    }
  }
}
