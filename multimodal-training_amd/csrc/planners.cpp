// Host-side integer planners of the vision tower (no device work).
// Closed-form index arithmetic; every function documents the reference span it replaces in
// include/mi355_vit.h.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/mi355_vit.h"

static thread_local char g_err[512] = "";

int mvit_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" {

int mvit_version(void) { return MVIT_VERSION; }
const char* mvit_last_error(void) { return g_err; }

static int check_grid(const int64_t* g, int64_t n, int merge) {
  if (!g || n < 0 || merge <= 0) return mvit_set_error(MVIT_ERR_ARG, "grid_thw: null pointer or bad sizes");
  for (int64_t i = 0; i < n; ++i) {
    const int64_t t = g[3 * i], h = g[3 * i + 1], w = g[3 * i + 2];
    if (t <= 0 || h <= 0 || w <= 0 || h % merge || w % merge)
      return mvit_set_error(MVIT_ERR_ARG, "grid_thw[%lld] = (%lld,%lld,%lld) must be positive with h, w multiples of %d",
                            (long long)i, (long long)t, (long long)h, (long long)w, merge);
  }
  return MVIT_OK;
}

int mvit_rot_pos_ids(const int64_t* grid_thw, int64_t n, int merge, int64_t* pos_ids) {
  if (int rc = check_grid(grid_thw, n, merge)) return rc;
  if (!pos_ids) return mvit_set_error(MVIT_ERR_ARG, "pos_ids is null");
  int64_t o = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t t = grid_thw[3 * i], h = grid_thw[3 * i + 1], w = grid_thw[3 * i + 2];
    const int64_t bw = w / merge, per_frame = h * w, unit = (int64_t)merge * merge;
    // token p of a frame: block b = p / unit (row-major over (h/merge, w/merge)), then (dy, dx) inside the block
    for (int64_t f = 0; f < t; ++f)
      for (int64_t p = 0; p < per_frame; ++p, ++o) {
        const int64_t b = p / unit, r = p % unit;
        pos_ids[2 * o] = (b / bw) * merge + r / merge;
        pos_ids[2 * o + 1] = (b % bw) * merge + r % merge;
      }
  }
  return MVIT_OK;
}

int mvit_window_index(const int64_t* grid_thw, int64_t n, int merge, int window_size, int patch_size,
                      int64_t* window_index, int32_t* cu_window, int64_t cu_cap, int64_t* n_cu) {
  if (int rc = check_grid(grid_thw, n, merge)) return rc;
  if (!window_index || !cu_window || !n_cu || cu_cap < 1) return mvit_set_error(MVIT_ERR_ARG, "null output or cu_cap < 1");
  if (patch_size <= 0 || window_size <= 0) return mvit_set_error(MVIT_ERR_ARG, "bad window/patch size");
  const int64_t win = window_size / merge / patch_size;
  if (win <= 0) return mvit_set_error(MVIT_ERR_ARG, "window_size %d too small for merge %d * patch %d", window_size, merge, patch_size);
  const int64_t unit = (int64_t)merge * merge;
  int64_t o = 0, base = 0, ncu = 0, total = 0;
  cu_window[ncu++] = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t t = grid_thw[3 * i], gh = grid_thw[3 * i + 1] / merge, gw = grid_thw[3 * i + 2] / merge;
    // Windows that hold at least one unit: ceil(g / win) per axis.  (The reference also enumerates a band
    // of empty windows when g divides evenly; those add repeated cumulative entries that it then drops.)
    const int64_t nh = (gh + win - 1) / win, nw = (gw + win - 1) / win;
    for (int64_t f = 0; f < t; ++f)
      for (int64_t wr = 0; wr < nh; ++wr)
        for (int64_t wc = 0; wc < nw; ++wc) {
          const int64_t r0 = wr * win, r1 = std::min(gh, r0 + win), c0 = wc * win, c1 = std::min(gw, c0 + win);
          for (int64_t r = r0; r < r1; ++r)
            for (int64_t c = c0; c < c1; ++c) window_index[o++] = base + (f * gh + r) * gw + c;
          total += (r1 - r0) * (c1 - c0) * unit;
          if (total > INT32_MAX) return mvit_set_error(MVIT_ERR_ARG, "sequence longer than int32");
          if (ncu >= cu_cap) return mvit_set_error(MVIT_ERR_ARG, "cu_window capacity %lld too small", (long long)cu_cap);
          cu_window[ncu++] = (int32_t)total;
        }
    base += t * gh * gw;
  }
  *n_cu = ncu;
  return MVIT_OK;
}

int mvit_cu_seqlens(const int64_t* grid_thw, int64_t n, int32_t* cu, int64_t cu_cap, int64_t* n_cu) {
  if (int rc = check_grid(grid_thw, n, 1)) return rc;
  if (!cu || !n_cu || cu_cap < 1) return mvit_set_error(MVIT_ERR_ARG, "null output or cu_cap < 1");
  int64_t k = 0, total = 0;
  cu[k++] = 0;
  for (int64_t i = 0; i < n; ++i)
    for (int64_t f = 0; f < grid_thw[3 * i]; ++f) {
      total += grid_thw[3 * i + 1] * grid_thw[3 * i + 2];
      if (total > INT32_MAX) return mvit_set_error(MVIT_ERR_ARG, "sequence longer than int32");
      if (k >= cu_cap) return mvit_set_error(MVIT_ERR_ARG, "cu capacity %lld too small", (long long)cu_cap);
      cu[k++] = (int32_t)total;
    }
  *n_cu = k;
  return MVIT_OK;
}

int mvit_sp_token_cuts(int64_t sample_len, int sp, int64_t* cuts) {
  if (sample_len < 0 || sp <= 0 || !cuts) return mvit_set_error(MVIT_ERR_ARG, "bad sample_len/sp/cuts");
  const int64_t q = sample_len / sp, r = sample_len % sp;
  for (int k = 0; k <= sp; ++k) cuts[k] = k * q + std::min<int64_t>(k, r);
  return MVIT_OK;
}

int mvit_sp_window_cuts(int64_t sample_len, int sp, const int64_t* window_lengths, int64_t n_windows,
                        int64_t* cut_pos, int64_t* cut_idx) {
  if (sp <= 0 || !cut_pos || !cut_idx) return mvit_set_error(MVIT_ERR_ARG, "bad sp or null outputs");
  if (!window_lengths || n_windows <= 0)
    return mvit_set_error(MVIT_ERR_ARG, "Window-based splitting requested but no window lengths were provided.");
  std::vector<int64_t> prefix(n_windows + 1, 0);
  for (int64_t i = 0; i < n_windows; ++i) {
    if (window_lengths[i] <= 0)
      return mvit_set_error(MVIT_ERR_ARG, "Encountered non-positive window length %lld while splitting sequence parallel chunks.",
                            (long long)window_lengths[i]);
    prefix[i + 1] = prefix[i] + window_lengths[i];
  }
  if (prefix[n_windows] != sample_len)
    return mvit_set_error(MVIT_ERR_ARG, "Window lengths do not sum to sample length: %lld vs expected %lld",
                          (long long)prefix[n_windows], (long long)sample_len);
  const int64_t np = n_windows + 1;
  cut_pos[0] = 0;
  cut_idx[0] = 0;
  int64_t last = 0;
  for (int step = 1; step < sp; ++step) {
    const int64_t want = sample_len * step / sp;
    // first boundary >= want, searched from the previous cut
    int64_t idx = std::lower_bound(prefix.begin() + last, prefix.end(), want) - prefix.begin();
    // leave at least one boundary for each of the remaining ranks where possible
    int64_t cap = np - (sp - step);
    cap = std::max<int64_t>(std::max(cap, last), 0);
    cap = std::min(cap, np - 1);
    idx = std::min(std::max(idx, last), cap);
    cut_pos[step] = prefix[idx];
    cut_idx[step] = idx;
    last = idx;
  }
  cut_pos[sp] = prefix[n_windows];
  cut_idx[sp] = n_windows;
  return MVIT_OK;
}

}  // extern "C"
