// nnvhip_affine_fc: Star.affineMap / FullyConnectedLayer.reach for one set or an array of sets - the dispatcher that
// chooses between the dense contraction, the contraction over kept rows, the tile kernel, the shared product of an
// array of neighbouring sets and the gather / row-sum passes for unit-vector columns.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "internal.h"
#include "mfma_tile.h"

namespace nnvhip {

// Wt(r, k) = W(r, k): the Mp x Kp column-major weights row-major (ld = Kp), 32 x 32 tiles through LDS
__global__ __launch_bounds__(256) void transpose_weights_kernel(const double* __restrict__ W, double* __restrict__ Wt, int Mp, int Kp) {
  __shared__ double tile[32][33];
  const int k0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  for (int i = threadIdx.y; i < 32; i += 8) {
    const int k = k0 + i, r = r0 + threadIdx.x;
    tile[i][threadIdx.x] = (k < Kp && r < Mp) ? W[r + (int64_t)k * Mp] : 0.0;
  }
  __syncthreads();
  for (int i = threadIdx.y; i < 32; i += 8) {
    const int r = r0 + i, k = k0 + threadIdx.x;
    if (r < Mp && k < Kp) Wt[(int64_t)r * Kp + k] = tile[threadIdx.x][i];
  }
}

}  // namespace nnvhip

using namespace nnvhip;

// Shared set-up of the affine layers: validates the input array, allocates one output arena with
// the sets back to back, and creates output handles that share constraints and predicate bounds
// with their inputs.
int nnvhip::make_affine_outputs(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, int64_t Nout,
                                std::vector<nnvhip_star*>* outs, bool* contiguous, int64_t* total_cols) {
  int64_t ldout = round_up(Nout, kLdAlign);
  int64_t cols = 0;
  bool contig = true;
  for (int64_t i = 0; i < count; ++i) {
    if (i > 0 && (in[i]->ld != in[0]->ld || in[i]->V != in[i - 1]->V + in[i - 1]->stored_cols() * in[i - 1]->ld)) contig = false;
    cols += in[i]->n + 1;
  }
  BufRef arena;
  NNV_TRY(c->alloc(sizeof(double) * ldout * cols, &arena));
  int64_t off = 0;
  for (int64_t i = 0; i < count; ++i) {
    nnvhip_star* o = new_star(c);
    o->N = Nout;
    o->n = in[i]->n;
    o->ld = ldout;
    o->Vbuf = arena;
    o->V = arena->as<double>() + off * ldout;
    o->pbuf = in[i]->pbuf;
    o->plb = in[i]->plb;
    o->pub = in[i]->pub;
    o->ptails = in[i]->ptails;
    o->pslot = in[i]->pslot;
    o->pcap = in[i]->pcap;
    o->cons = in[i]->cons;
    off += in[i]->n + 1;
    outs->push_back(o);
  }
  *contiguous = contig;
  *total_cols = cols;
  return NNVHIP_OK;
}

void nnvhip::release_all(std::vector<nnvhip_star*>& v) {
  for (auto* s : v) nnvhip_star_release(s);
  v.clear();
}

int nnvhip::check_set_array(nnvhip_ctx* c, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  if (!in || !out || count <= 0) NNV_FAIL(NNVHIP_ERR_ARG, "null argument");
  for (int64_t i = 0; i < count; ++i)
    if (!in[i] || in[i]->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid set handle %lld", (long long)i);
  return NNVHIP_OK;
}
extern "C" {

int nnvhip_affine_fc(nnvhip_ctx* c, const nnvhip_fc* fc, int64_t count, nnvhip_star* const* in, nnvhip_star** out) {
  CHECK_CTX(c);
  if (!fc || fc->ctx != c) NNV_FAIL(NNVHIP_ERR_ARG, "invalid layer handle");
  NNV_TRY(check_set_array(c, count, in, out));
  for (int64_t i = 0; i < count; ++i)
    if (in[i]->N != fc->K)
      NNV_FAIL(NNVHIP_ERR_SHAPE, "Inconsistency between the affine mapping matrix and dimension of the star set");
  std::vector<nnvhip_star*> outs;
  bool contig = false;
  int64_t cols = 0;
  NNV_TRY(c->begin_op());
  // A large array whose gathered columns will stay unwritten gets their range sums from one matrix product
  // (see below).  Nothing of it depends on the outputs, so it is queued before anything else: the device
  // works on it while the host sets up the outputs and the tiles of the contraction.
  BufRef mm_early;
  std::vector<int64_t> mm_slot;  // which pair of the product's columns holds a set's sums
  bool mm_plb_zero = true;       // every gathered column of every set has predicate lower bound 0
  int st = NNVHIP_OK;
  if (count >= 64 && !c->eager_cols && !c->dense_affine) {
    std::vector<GatherSet> es((size_t)count);
    bool ok = true, any = false;
    for (int64_t i = 0; i < count; ++i) {
      const int64_t nc = in[i]->n + 1;
      int64_t d = (in[i]->oh_from > 0 && in[i]->oh_from < nc) ? in[i]->oh_from : nc;
      if ((double)fc->Mp * (double)fc->Kp * (double)(nc - d) * (double)count < 4.0e6) d = nc;
      GatherSet& g = es[i];
      g = GatherSet{};
      g.idx = in[i]->oh_idx;
      g.scale = in[i]->oh_scale;
      g.plb = in[i]->plb + (d - 1);  // the output shares the input's predicate bounds
      g.pub = in[i]->pub + (d - 1);
      g.m = (int32_t)(nc - d);
      ok = ok && !(g.m > 0 && in[i]->oh_scale_neg);
      any = any || g.m > 0;
      mm_plb_zero = mm_plb_zero && (g.m == 0 || in[i]->oh_plb_zero);
    }
    // (the ReLU step that made the sets may have queued this very product already: nnvhip_hint_next_fc)
    bool ahead = ok && any && mm_plb_zero;
    for (int64_t i = 0; i < count && ahead; ++i)
      ahead = in[i]->ahead_mm_buf && in[i]->ahead_mm_uid == fc->uid && in[i]->ahead_mm_buf == in[0]->ahead_mm_buf &&
              in[i]->oh_scale == nullptr;
    if (ahead) {
      mm_early = in[0]->ahead_mm_buf;
      mm_slot.resize((size_t)count);
      for (int64_t i = 0; i < count; ++i) mm_slot[(size_t)i] = in[i]->ahead_mm_slot;
    } else if (ok && any) {
      st = launch_range_sums_mm(c, fc, count, es.data(), &mm_early, &mm_slot, mm_plb_zero);
    }
  }
  if (st == NNVHIP_OK) st = make_affine_outputs(c, count, in, fc->M, &outs, &contig, &cols);
  if (st == NNVHIP_OK) {
    for (int64_t i = 0; i < count; ++i) outs[i]->has_zono = in[i]->has_zono;  // Z.affineMap(W, b), set/Star.m:332-340
    const double* bias = fc->bias ? fc->bias->as<double>() : nullptr;
    const double* Wd = fc->W->as<double>();
    // Columns of V that are scaled unit vectors (all generators of a box star, the columns a ReLU
    // appended) need no contraction: W * (s * e_r) = s * W(:, r).  dense[i] = leading columns that do.
    const bool dense_only = c->dense_affine;
    std::vector<int64_t> dense((size_t)count);
    std::vector<GatherSet> gs((size_t)count);
    int64_t total_dense = 0;
    bool any_onehot = false;
    for (int64_t i = 0; i < count; ++i) {
      const int64_t nc = in[i]->n + 1;
      dense[i] = (!dense_only && in[i]->oh_from > 0 && in[i]->oh_from < nc) ? in[i]->oh_from : nc;
      // tiny products are launch bound: one dense launch beats GEMM + gather
      if ((double)fc->Mp * (double)fc->Kp * (double)(nc - dense[i]) * (double)count < 4.0e6) dense[i] = nc;
      total_dense += dense[i];
      any_onehot = any_onehot || dense[i] < nc;
      GatherSet& g = gs[i];
      g.idx = in[i]->oh_idx;
      g.scale = in[i]->oh_scale;
      g.out = outs[i]->V + dense[i] * outs[i]->ld;
      g.plb = outs[i]->plb + (dense[i] - 1);
      g.pub = outs[i]->pub + (dense[i] - 1);
      g.part = nullptr;
      g.m = (int32_t)(nc - dense[i]);
      g.nfill = 0;
      g.fill = nullptr;
      g.bias = nullptr;
      g.red = nullptr;
      g.red_k = 0;
      g.lazy = 0;
      g.cin = nullptr;
      g.cpart = nullptr;
      g.centre = nullptr;
    }
    // One set whose gathered columns can stay unwritten and are either all the generators of a box star or the
    // columns a ReLU step appended (with that step's per-row classes still on the handle): the output's lb / ub
    // come from launch_fc_rowsum: one kernel over the weights instead of a gather pass plus a reduction.
    const bool lazy_ok = !c->eager_cols && !dense_only;
    const bool box_in = count == 1 && in[0]->oh_from == 1 && in[0]->oh_scale != nullptr && !in[0]->oh_scale_neg && dense[0] == 1 &&
                        gs[0].m > 0;
    const bool relu_in = count == 1 && in[0]->oh_from > 1 && in[0]->oh_scale == nullptr && gs[0].m > 0 && dense[0] == in[0]->oh_from &&
                         in[0]->rows_pending && in[0]->cls != nullptr && in[0]->pre_ub != nullptr;
    // (skinny layers keep the gather pass: a handful of 16-row blocks would not cover the chip)
    bool rowsum = (box_in || relu_in) && fc->Mp >= 128 && fc->K < (int64_t(1) << 31);
    // sets whose implicit unit-vector columns take part in the contraction after all get them written out
    // (which also runs a pending row reset)
    std::vector<nnvhip_star*> full;
    for (int64_t i = 0; i < count; ++i)
      if (dense[i] > in[i]->stored_cols() || (dense_only && (in[i]->rows_pending || in[i]->cs.any_pending()))) full.push_back(in[i]);
    if (!full.empty()) {
      st = ensure_dense_batch(c, (int64_t)full.size(), full.data());
      contig = true;  // the sets moved: look again
      for (int64_t i = 1; i < count; ++i)
        if (in[i]->ld != in[0]->ld || in[i]->V != in[i - 1]->V + in[i - 1]->stored_cols() * in[i - 1]->ld) contig = false;
    }
    // Matrices a shared-product call left unwritten (ColSource::delta) are written before rows of them are read; a set
    // that keeps no row reads none.
    {
      std::vector<nnvhip_star*> need;
      for (int64_t i = 0; i < count; ++i)
        if (in[i]->cs.delta_pending() && !(in[i]->rows_pending && in[i]->n_kept == 0)) need.push_back(in[i]);
      if (!need.empty() && st == NNVHIP_OK) st = write_pending_columns(c, (int64_t)need.size(), need.data());
    }
    // Rows of the dense columns that the ReLU step reset to zero need no contraction either: the
    // GEMM then runs over the kept rows only (used when that at least halves K).
    // *pack: gather the listed rows into a matrix of their own first (several row tiles of W would each
    // gather them otherwise; and a long list read through the map is slow, so a set that only takes this
    // route because its reset is pending always packs)
    auto rows_of = [&](int64_t i, GemmRows* r, int64_t* kp, bool* pack) {
      *kp = fc->Kp;
      *pack = fc->Mp > 128;
      // a set whose row reset is still pending shares its matrix with the ReLU's input: only the listed
      // rows may be read
      const bool must = in[i]->rows_pending;
      if (!must && (dense_only || in[i]->n_kept < 0 || in[i]->kept_idx == nullptr)) return false;
      // the kept-row list describes the columns before the one-hot block only (a one-hot column has its
      // 1 in a reset row): usable only if that block is not part of the contraction
      if (in[i]->oh_from > 0 && dense[i] > in[i]->oh_from) return false;
      const bool tiny = (double)fc->Mp * (double)fc->Kp * (double)dense[i] * (double)count < 4.0e6;
      if (!must && tiny) return false;
      const int64_t k = std::max<int64_t>(round_up(in[i]->n_kept, kLdAlign), kLdAlign);
      if (!must && 2 * k > fc->Kp) return false;
      if (tiny)
        *pack = false;  // launch bound: read through the map
      else if (must && 2 * k > fc->Kp)
        *pack = true;
      r->kmap = in[i]->kept_idx;
      r->flop = 2.0 * (double)fc->Mp * (double)k * (double)dense[i];
      *kp = k;
      return true;
    };
    // A set whose kept-row list is empty contracts over nothing: its dense columns are the bias and
    // zeros, which the gather pass writes along with its own columns (no GEMM, no packing).
    auto nothing_kept = [&](int64_t i, const GemmRows& r) { return r.kmap != nullptr && in[i]->n_kept == 0; };
    auto fill_by_gather = [&](int64_t i) {
      gs[i].nfill = (int32_t)dense[i];
      gs[i].fill = outs[i]->V;
      gs[i].bias = bias;
    };
    // Inputs with columns that are described but not in memory yet: the contraction reads them from
    // memory unless it goes over no row at all or through the packing pass (which takes such columns
    // from the weights they were gathered from).  Everybody else has them written now.
    if (st == NNVHIP_OK) {
      std::vector<nnvhip_star*> cols;
      for (int64_t i = 0; i < count; ++i) {
        if (!in[i]->cs.any_pending()) continue;
        GemmRows r;
        int64_t kp = 0;
        bool pack = false;
        const bool compact = rows_of(i, &r, &kp, &pack);
        if (!(compact && (nothing_kept(i, r) || (pack && r.kmap != nullptr)))) cols.push_back(in[i]);
      }
      if (!cols.empty()) st = write_pending_columns(c, (int64_t)cols.size(), cols.data());
    }
    // Gathered columns whose range sums this call leaves behind are not written: the ReLU step that
    // follows works from the sums, and the next FC map either contracts over no row or packs its rows
    // from the weights.  lazy[i] is set where the sums are produced.
    std::vector<char> lazy((size_t)count, 0);
    if (count == 1 && rowsum && st == NNVHIP_OK) {
      GemmRows rows;
      int64_t kp = fc->Kp;
      bool pack = false;
      const bool compact = rows_of(0, &rows, &kp, &pack);
      const int mode = box_in ? 0 : 1;
      if (box_in) {
        // the centre's product W * c + b is formed along the way: no GEMM launch at all
        st = launch_fc_rowsum(c, fc, outs[0], mode, in[0]->oh_scale, nullptr, nullptr, 1, in[0]->V, nullptr, 0);
        lazy[0] = lazy_ok;
      } else if (compact && nothing_kept(0, rows)) {
        // no row kept: the contracted columns are the bias and zeros, of which only the centre is stored
        fill_by_gather(0);
        st = launch_fc_rowsum(c, fc, outs[0], mode, nullptr, in[0]->cls, in[0]->pre_ub, 2, nullptr, nullptr, 0);
        lazy[0] = lazy_ok;
      } else {
        RangeFuse fuse;
        fuse.plb = outs[0]->plb;
        fuse.pub = outs[0]->pub;
        BufRef packed;
        // enough 128 x 128 tiles to go round: the tile kernel of gemm_seg.hip (rows packed transposed, operands
        // staged straight into LDS), as for an array of sets
        const int64_t tiles128 = ceil_div(dense[0], 128) * ceil_div(fc->Mp, 128);
        const bool tile_kernel = compact && pack && rows.kmap != nullptr && !dense_only && tiles128 >= 128 && kp <= 2048 &&
                                 dense[0] < (int64_t(1) << 24);
        if (tile_kernel) {
          const int64_t ldo = outs[0]->ld, ldt = round_up(dense[0], 128), ntiles = ceil_div(dense[0], 128);
          st = c->alloc(sizeof(double) * kp * ldt, &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            ps.ldt = ldt;
            st = launch_pack_rows_t(c, 1, &ps);
          }
          if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * 4 * ldo * ntiles, &fuse.part);
          fuse.chunks = ntiles;
          // tiles by width: [0] 128 columns, [1] 64, [2] 32 (the last tile, if the remainder fits)
          std::vector<SegTile> tiles[3];
          double flop[3] = {0.0, 0.0, 0.0};
          for (int64_t j = 0; j < dense[0] && st == NNVHIP_OK; j += 128) {
            const int64_t valid = std::min<int64_t>(128, dense[0] - j);
            const int w = valid > 64 ? 0 : valid > 32 ? 1 : 2;
            SegTile sg{};
            sg.kmap = rows.kmap;
            sg.Bt = packed->as<double>();
            sg.ldbt = ldt;
            sg.b_col0 = j;
            sg.col_local0 = j;
            sg.col_base = j;
            sg.kp = (int32_t)kp;
            sg.valid = (int32_t)valid;
            sg.plb = outs[0]->plb;
            sg.pub = outs[0]->pub;
            sg.rpart = fuse.part->as<double>() + 4 * ldo * (j / 128);
            tiles[w].push_back(sg);
            flop[w] += 2.0 * (double)fc->Mp * (double)kp * (double)valid;
          }
          static const int widths[3] = {128, 64, 32};
          for (int w = 0; w < 3 && st == NNVHIP_OK; ++w) {
            if (tiles[w].empty()) continue;
            BufRef dt;
            st = c->upload_table(tiles[w].data(), sizeof(SegTile) * tiles[w].size(), &dt);
            if (st == NNVHIP_OK)
              st = launch_gemm_seg(c, Wd, fc->Mp, outs[0]->V, ldo, fc->Mp, bias, widths[w], dt->as<SegTile>(), (int64_t)tiles[w].size(),
                                   flop[w]);
          }
        } else if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[0], &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            st = launch_pack_rows(c, 1, &ps);
            rows.Bk = packed->as<double>();
            rows.ldbk = kp;
          }
        }
        if (st == NNVHIP_OK && !tile_kernel)
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, dense[0], kp, bias, &fuse,
                           compact ? &rows : nullptr);
        if (st == NNVHIP_OK && fuse.chunks > 0) {
          st = launch_fc_rowsum(c, fc, outs[0], mode, nullptr, in[0]->cls, in[0]->pre_ub, 0, nullptr, fuse.part->as<double>(), fuse.chunks);
          lazy[0] = lazy_ok;
        } else if (st == NNVHIP_OK) {
          // the product was split along K and left no sums: the columns are written
          if (st == NNVHIP_OK) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), 0);
        }
      }
      // a caller that wants the gathered columns in memory gets them written now (same values as a later
      // first read would write)
      if (st == NNVHIP_OK && outs[0]->lb != nullptr && !lazy_ok) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), 0);
    } else if (count == 1) {
      // one set: the GEMM epilogue also leaves the partial sums of Star.estimateRanges, so the
      // output set carries its ranges without another pass over V
      RangeFuse fuse;
      fuse.plb = outs[0]->plb;
      fuse.pub = outs[0]->pub;
      const int64_t gch = gather_chunks(fc->Mp, gs[0].m);
      fuse.extra_chunks = gch;
      GemmRows rows;
      int64_t kp = fc->Kp;
      bool pack = false;
      const bool compact = rows_of(0, &rows, &kp, &pack);
      if (compact && nothing_kept(0, rows)) {
        fill_by_gather(0);
        const int64_t ch = std::max<int64_t>(1, gather_chunks(fc->Mp, std::max<int64_t>(gs[0].m, gs[0].nfill)));
        BufRef part;
        if (gs[0].m > 0) {
          st = c->alloc(sizeof(double) * 4 * outs[0]->ld * ch, &part);
          if (st == NNVHIP_OK) gs[0].part = part->as<double>();
          lazy[0] = lazy_ok;
          gs[0].lazy = lazy[0];
        }
        if (st == NNVHIP_OK) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), gs[0].m > 0 ? ch : 0);
        if (st == NNVHIP_OK && gs[0].m > 0) st = finalize_fused_ranges(c, outs[0], part, ch);
      } else {
        BufRef packed;
        if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[0], &packed);
          if (st == NNVHIP_OK) {
            PackSet ps = pack_of(in[0], in[0]->kept_idx, packed->as<double>(), kp, dense[0]);
            st = launch_pack_rows(c, 1, &ps);
            rows.Bk = packed->as<double>();
            rows.ldbk = kp;
          }
        }
        // only the centre is contracted (a box star): the range sums are the gather's alone
        const bool centre_only = dense[0] == 1 && gs[0].m > 0;
        // ... and when the gathered columns are all the columns of W (no degenerate dimension), the gather
        // pass forms the centre's product as well, one partial vector per chunk: no GEMM launch at all
        const bool centre_in_gather = centre_only && !compact && gs[0].m == fc->K && in[0]->oh_from == 1 && gch > 0;
        SplitKDefer defer;  // (otherwise the gather pass sums the centre's split-K partials)
        BufRef cpart;
        if (st == NNVHIP_OK && centre_in_gather) {
          st = c->alloc(sizeof(double) * outs[0]->ld * gch, &cpart);
          if (st == NNVHIP_OK) {
            gs[0].cin = in[0]->V;
            gs[0].cpart = cpart->as<double>();
          }
        } else if (st == NNVHIP_OK) {
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, dense[0], kp, bias,
                           centre_only ? nullptr : &fuse, compact ? &rows : nullptr, centre_only ? &defer : nullptr);
        }
        if (st == NNVHIP_OK && centre_only) {
          st = c->alloc(sizeof(double) * 4 * outs[0]->ld * gch, &fuse.part);
          fuse.chunks = 0;
          if (defer.ksplit > 1) {
            gs[0].red = defer.ws->as<double>();
            gs[0].red_k = (int32_t)defer.ksplit;
            gs[0].centre = outs[0]->V;
            gs[0].bias = bias;
          }
        }
        const bool fused = st == NNVHIP_OK && (fuse.chunks > 0 || centre_only);
        if (st == NNVHIP_OK && gs[0].m > 0) {
          gs[0].part = fused ? fuse.part->as<double>() + fuse.chunks * 4 * outs[0]->ld : nullptr;
          lazy[0] = lazy_ok && fused;
          gs[0].lazy = lazy[0];
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[0]->ld, 1, gs.data(), fused ? gch : 0);
        }
        if (st == NNVHIP_OK && fused)
          st = finalize_fused_ranges(c, outs[0], fuse.part, fuse.chunks + (gs[0].m > 0 ? gch : 0),
                                     centre_in_gather ? cpart->as<double>() : nullptr, centre_in_gather ? gch : 0, bias);
      }
    } else if (contig) {
      // one launch for the whole array.  With structure to exploit, every set's dense columns are cut
      // into tiles of 128 that carry their own description (row list, position in the arena).
      bool any_rows = false, bias_in_kernel = false;
      std::vector<GemmRows> rws((size_t)count);
      std::vector<int64_t> kps((size_t)count);
      std::vector<char> pk((size_t)count, 0);
      std::vector<char> filled((size_t)count, 0);
      bool any_fill = false;
      // Range sums: chunk_off[i] .. chunk_off[i+1] are set i's chunks of [4][ld] partial sums in `sums`,
      // first one per column tile of the segmented GEMM (tiles_of[i], filled by its epilogue), then the
      // gather pass's gch chunks if the set has gathered columns.
      BufRef sums;
      std::vector<int64_t> tiles_of((size_t)count, 0), chunk_off((size_t)count + 1, 0);
      int64_t gch = 0;
      {
        int64_t max_m = 0;
        for (int64_t i = 0; i < count; ++i) max_m = std::max<int64_t>(max_m, gs[i].m);
        gch = gather_chunks_batch(outs[0]->ld, count, max_m);  // 0: nothing to gather
      }
      // large arrays: the sums of the gathered columns come from one matrix product instead (gch_part = 0:
      // the gather pass leaves no chunks)
      bool use_mm = lazy_ok && gch > 0 && count >= 64;
      for (int64_t i = 0; i < count; ++i) use_mm = use_mm && !(gs[i].m > 0 && in[i]->oh_scale_neg);
      const int64_t gch_part = use_mm ? 0 : gch;
      BufRef mm_sums;
      for (int64_t i = 0; i < count; ++i) {
        bool pack = false;
        any_rows = rows_of(i, &rws[i], &kps[i], &pack) || any_rows;
        pk[i] = pack && rws[i].kmap != nullptr;
        if (nothing_kept(i, rws[i])) {
          fill_by_gather(i);
          filled[i] = 1;
          pk[i] = 0;
          any_fill = true;
        }
      }
      bool all_stored = true;
      for (int64_t i = 0; i < count; ++i) all_stored = all_stored && in[i]->stored_cols() == in[i]->n + 1;
      if (any_onehot && !any_rows && all_stored) {
        // all sets contract over every row: their dense columns are simply listed (tiles may span sets)
        if (cols >= (int64_t(1) << 31)) st = NNVHIP_ERR_SHAPE;
        std::vector<int32_t> map;
        map.reserve((size_t)total_dense);
        int64_t off = 0;
        for (int64_t i = 0; i < count; ++i) {
          for (int64_t j = 0; j < dense[i]; ++j) map.push_back((int32_t)(off + j));
          off += in[i]->n + 1;  // box stars: all columns stored, input and output arenas laid out alike
        }
        BufRef cmap;
        if (st == NNVHIP_OK) st = c->upload_table(map.data(), sizeof(int32_t) * map.size(), &cmap);
        if (st == NNVHIP_OK) {
          GemmRows rows;
          rows.colmap = cmap->as<int32_t>();
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, total_dense, fc->Kp, bias,
                           nullptr, &rows);
        }
      } else if (any_rows || any_onehot) {
        std::vector<GemmSeg> segs;
        GemmRows rows;
        const int64_t tn = gemm_seg_cols(fc->Mp, count, dense.data());
        rows.seg_cols = (int32_t)tn;
        // Large arrays whose sets all come with packed rows take the tile kernel of gemm_seg.hip: rows packed
        // transposed, operands staged straight into LDS, a narrow last tile per set, bias added in the kernel.
        bool seg_tiles = tn == 128 && !dense_only;
        for (int64_t i = 0; i < count; ++i)
          if (!filled[i] && (!pk[i] || kps[i] > 2048 || dense[i] >= (int64_t(1) << 24))) seg_tiles = false;
        if (seg_tiles) {
          const int64_t ldo = outs[0]->ld;
          BufRef packed, shared_rows;
          std::vector<PackSet> packs;
          std::vector<const double*> bt((size_t)count, nullptr);
          std::vector<int64_t> ldt((size_t)count, 0);
          // Sets whose generator columns are all the same scaled weight columns (boxes of one shape through an FC
          // layer and a ReLU: same index list, same scales) have the same packed rows wherever they keep the same
          // row.  One matrix then serves them all - row r = what any of them would pack for input row r - and the
          // 128-column tiles gather its rows through their own kept-row lists; only a set's centre column (patched
          // in by its first tile) and the columns past the last whole tile (packed as before) are its own.
          struct RowShape {  // what decides a set's packed rows besides its kept-row list
            const double* Wt;
            int64_t ldwt, rows;
            const int32_t* idx;
            const double* scale;
            int64_t dense, ldws, nfull, off;
          };
          std::vector<RowShape> shapes;
          std::vector<int> shape_of((size_t)count, -1);
          bool shared = true;
          for (int64_t i = 0; i < count && shared; ++i) {
            if (filled[i]) continue;
            const ColSource& cs = in[i]->cs;
            shared = cs.W != nullptr && cs.Wt != nullptr && cs.from == 1 && cs.from + cs.cols >= dense[i] && cs.zero_to <= 1 &&
                     !cs.win_pending() && dense[i] >= 128 && cs.rows < (int64_t(1) << 30);
            if (!shared) break;
            for (size_t k = 0; k < shapes.size() && shape_of[i] < 0; ++k) {
              const RowShape& r = shapes[k];
              if (r.Wt == cs.Wt && r.ldwt == cs.ldwt && r.rows == cs.rows && r.idx == cs.idx && r.scale == cs.scale && r.dense == dense[i])
                shape_of[i] = (int)k;
            }
            if (shape_of[i] < 0) {
              if (shapes.size() == 16) {  // too many different shapes for the matrices to pay
                shared = false;
                break;
              }
              shape_of[i] = (int)shapes.size();
              shapes.push_back(RowShape{cs.Wt, cs.ldwt, cs.rows, cs.idx, cs.scale, dense[i], round_up(dense[i], 128), dense[i] / 128, 0});
            }
          }
          shared = shared && !shapes.empty();
          // Sets of one shape differ in their products only through their kept-row lists (and their centres).  Where
          // the lists of a group are nearly the same - the sub-boxes of one box, whose first-layer bounds differ by
          // little - the group's product over the rows most of its sets keep is formed once (by the tile kernel), and a
          // set's output is that product plus the few rows in which the set differs, written by one streaming pass
          // (delta_try / delta_done below).
          bool delta_try = shared && count >= 32 && !c->no_row_deltas;
          for (size_t k = 1; k < shapes.size() && delta_try; ++k) delta_try = shapes[k].rows == shapes[0].rows;
          delta_try = delta_try && !shapes.empty() && shapes[0].rows == fc->Kp && shapes[0].rows < (int64_t(1) << 20);
          if (shared) {
            int64_t doubles = 0;
            for (RowShape& r : shapes) {
              r.off = doubles;
              doubles += (r.rows + 1) * r.ldws;
            }
            st = c->alloc(sizeof(double) * doubles, &shared_rows);
            ScaledRows sr{};
            for (size_t k = 0; k < shapes.size(); ++k) {
              const RowShape& r = shapes[k];
              sr.s[k] = ScaledRows::One{r.Wt, r.ldwt, r.idx, r.scale, shared_rows ? shared_rows->as<double>() + r.off : nullptr, r.ldws,
                                        (int32_t)r.rows, (int32_t)r.dense};
            }
            sr.count = (int32_t)shapes.size();
            if (st == NNVHIP_OK) st = launch_scaled_rows(c, sr);
          }
          bool delta_done = false;
          if (delta_try && st == NNVHIP_OK) {
            constexpr int kDeltaCap = 64;
            const int groups = (int)shapes.size();
            const int64_t rowsK = shapes[0].rows, rows_pad = round_up(rowsK, 16);
            std::vector<int64_t> act;  // the sets that take part (not filled)
            std::vector<DeltaSet> dsets;
            std::vector<CentreSet> csets;
            std::vector<int32_t> gsize((size_t)groups, 0);
            for (int64_t i = 0; i < count; ++i)
              if (!filled[i]) {
                act.push_back(i);
                dsets.push_back(DeltaSet{rws[i].kmap, (int32_t)kps[i], (int32_t)shape_of[i]});
                csets.push_back(CentreSet{rws[i].kmap, in[i]->V, (int32_t)kps[i]});
                gsize[(size_t)shape_of[i]]++;
              }
            const int64_t nact = (int64_t)act.size();
            BufRef dtab, ctab, gtab, votes, common, lens, delta;
            if (nact == 0) st = NNVHIP_OK;
            if (nact > 0) {
              st = c->upload_table(dsets.data(), sizeof(DeltaSet) * dsets.size(), &dtab);
              if (st == NNVHIP_OK) st = c->upload_table(gsize.data(), sizeof(int32_t) * gsize.size(), &gtab);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * groups * rowsK, &votes);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * groups * rows_pad, &common);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * (groups + 5 * nact), &lens);  // ncommon, dlen, first entries
              if (st == NNVHIP_OK) st = c->alloc(sizeof(int32_t) * nact * kDeltaCap, &delta);
              if (st == NNVHIP_OK)
                st = launch_delta_lists(c, nact, dtab->as<DeltaSet>(), groups, gtab->as<int32_t>(), rowsK, rows_pad, kDeltaCap,
                                        votes->as<int32_t>(), common->as<int32_t>(), lens->as<int32_t>(), delta->as<int32_t>(),
                                        lens->as<int32_t>() + groups, lens->as<int32_t>() + groups + nact);
              // the lengths of the lists come back, and with them the first four entries of each (what the sets are
              // put in order by further down)
              // While they travel and the host sets the tiles up, the device forms what does not depend on them: the
              // centres, which are the sets' own - W * (centre masked to the kept rows), all sets in one product
              // (wasted where the lists turn out too long for this route, next to the much longer work that follows
              // then).
              std::vector<int32_t> hl((size_t)(groups + nact)), head((size_t)(4 * nact));
              BufRef cm, cprod;
              if (st == NNVHIP_OK) st = c->upload_table(csets.data(), sizeof(CentreSet) * csets.size(), &ctab);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * fc->Kp * nact, &cm);
              if (st == NNVHIP_OK) st = c->alloc(sizeof(double) * fc->Mp * nact, &cprod);
              if (st == NNVHIP_OK) {
                void* hp = nullptr;
                st = c->stage(sizeof(int32_t) * (hl.size() + head.size()), &hp);
                if (st == NNVHIP_OK) {
                  int32_t* hh = static_cast<int32_t*>(hp) + hl.size();
                  if (hipMemcpyAsync(hp, lens->ptr, sizeof(int32_t) * (hl.size() + head.size()), hipMemcpyDeviceToHost, c->stream) !=
                          hipSuccess ||
                      hipEventRecord(c->read_ev, c->stream) != hipSuccess) {
                    set_error("HIP error reading the row-difference lists back");
                    st = NNVHIP_ERR_HIP;
                  }
                  if (st == NNVHIP_OK) st = launch_masked_centres(c, nact, ctab->as<CentreSet>(), cm->as<double>(), fc->Kp);
                  if (st == NNVHIP_OK)
                    st = launch_gemm(c, Wd, fc->Mp, cm->as<double>(), fc->Kp, cprod->as<double>(), fc->Mp, fc->Mp, nact, fc->Kp, nullptr);
                  if (st == NNVHIP_OK && hipEventSynchronize(c->read_ev) != hipSuccess) {
                    set_error("HIP error reading the row-difference lists back");
                    st = NNVHIP_ERR_HIP;
                  }
                  if (st == NNVHIP_OK) {
                    memcpy(hl.data(), hp, sizeof(int32_t) * hl.size());
                    memcpy(head.data(), hh, sizeof(int32_t) * head.size());
                  }
                }
              }
              bool fits = st == NNVHIP_OK;
              int64_t delta_rows = 0;
              for (int64_t a = 0; a < nact && fits; ++a) {
                fits = hl[(size_t)(groups + a)] >= 0;
                delta_rows += std::max<int32_t>(hl[(size_t)(groups + a)], 0);
              }
              // worth it when a set's differences are a small part of its list
              int64_t kept_rows = 0;
              for (int64_t a = 0; a < nact; ++a) kept_rows += kps[act[(size_t)a]];
              fits = fits && 4 * delta_rows <= kept_rows;
              if (fits) {
                const int64_t ldo = outs[0]->ld, Mp = fc->Mp;
                // the groups' shared products: the same tiles, over the majority lists, into a buffer of their own
                int64_t base_cols = 0;
                std::vector<int64_t> base_off((size_t)groups);
                for (int g = 0; g < groups; ++g) {
                  base_off[(size_t)g] = base_cols;
                  base_cols += shapes[(size_t)g].ldws;
                }
                BufRef basebuf;
                st = c->alloc(sizeof(double) * Mp * base_cols, &basebuf);
                std::vector<SegTile> bt_tiles;
                double base_flop = 0.0;
                for (int g = 0; g < groups && st == NNVHIP_OK; ++g) {
                  const RowShape& r = shapes[(size_t)g];
                  if (gsize[(size_t)g] == 0) continue;
                  for (int64_t j = 0; j < r.dense; j += 128) {
                    SegTile sg{};
                    sg.kmap = common->as<int32_t>() + (int64_t)g * rows_pad;
                    sg.Bt = shared_rows->as<double>() + r.off;
                    sg.ldbt = r.ldws;
                    sg.b_col0 = j;
                    sg.col_local0 = j;
                    sg.col_base = base_off[(size_t)g] + j;
                    sg.gather_b = 1;
                    sg.zero_row = (int32_t)r.rows;
                    sg.kp = hl[(size_t)g];
                    sg.valid = (int32_t)std::min<int64_t>(128, r.dense - j);
                    bt_tiles.push_back(sg);
                    base_flop += 2.0 * (double)Mp * (double)sg.kp * (double)sg.valid;
                  }
                }
                if (st == NNVHIP_OK && !bt_tiles.empty()) {
                  BufRef dt;
                  st = c->upload_table(bt_tiles.data(), sizeof(SegTile) * bt_tiles.size(), &dt);
                  if (st == NNVHIP_OK)
                    st = launch_gemm_seg(c, Wd, Mp, basebuf->as<double>(), Mp, Mp, nullptr, 128, dt->as<SegTile>(), (int64_t)bt_tiles.size(),
                                         base_flop, true);
                }
                // the sets' tiles, by column tile and group so that tiles that read the same piece of a shared product
                // run next to one another
                for (int64_t i = 0; i < count; ++i) {
                  tiles_of[i] = filled[i] ? 0 : delta_tile_chunks(dense[i]);
                  chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
                }
                if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
                std::vector<int64_t> col_off((size_t)count, 0);
                {
                  int64_t off = 0;
                  for (int64_t i = 0; i < count; ++i) {
                    col_off[(size_t)i] = off;
                    off += in[i]->n + 1;
                  }
                }
                // the sets by group, so that neighbours in the table read the same shared product
                std::vector<DeltaOut> douts;
                std::vector<int64_t> dset;  // the set each entry of the table is
                std::vector<int32_t> dgroup;
                double dbytes = 0.0;
                int64_t max_cols = 0;
                // (within a group by the length of their lists and by the lists' first entries: sets with the same list -
                // those without differences, whose pieces are the shared product itself, above all - then stand next to
                // one another, and the pass that stores nothing sums a piece once for a run of sets that agree in list
                // and bounds)
                std::vector<int64_t> order;
                for (int g = 0; g < groups; ++g) {
                  const size_t from = order.size();
                  for (int64_t a = 0; a < nact; ++a)
                    if (shape_of[act[(size_t)a]] == g) order.push_back(a);
                  std::stable_sort(order.begin() + (int64_t)from, order.end(), [&](int64_t x, int64_t y) {
                    const int32_t lx = hl[(size_t)(groups + x)], ly = hl[(size_t)(groups + y)];
                    if (lx != ly) return lx < ly;
                    for (int t = 0; t < std::min(lx, 4); ++t)
                      if (head[(size_t)(4 * x + t)] != head[(size_t)(4 * y + t)]) return head[(size_t)(4 * x + t)] < head[(size_t)(4 * y + t)];
                    return false;
                  });
                }
                for (size_t k = 0; k < order.size() && st == NNVHIP_OK; ++k) {
                  const int64_t a = order[k];
                  const int64_t i = act[(size_t)a];
                  const int g = shape_of[i];
                  const RowShape& r = shapes[(size_t)g];
                  DeltaOut d{};
                  d.delta = delta->as<int32_t>() + a * kDeltaCap;
                  d.base = basebuf->as<double>() + base_off[(size_t)g] * Mp;
                  d.S = shared_rows->as<double>() + r.off;
                  d.lds = r.ldws;
                  d.cprod = cprod->as<double>() + a * Mp;
                  d.out = outs[0]->V + col_off[(size_t)i] * ldo;
                  d.plb = outs[i]->plb;
                  d.pub = outs[i]->pub;
                  d.rpart = sums->as<double>() + 4 * ldo * chunk_off[i];
                  d.dlen = hl[(size_t)(groups + a)];
                  d.ncols = (int32_t)dense[i];
                  douts.push_back(d);
                  dset.push_back(i);
                  dgroup.push_back((int32_t)g);
                  dbytes += 8.0 * (double)Mp * (double)dense[i];
                  max_cols = std::max<int64_t>(max_cols, dense[i]);
                }
                // Nothing on the way to the next layers reads these matrices where the layer's caller reads bounds only
                // (the ReLU step takes the range sums, the next FC layer the rows the step keeps - often none): unless
                // every column is to be in memory after the call, the pass forms and sums the pieces without storing
                // them, and the description stays on the handles (ColSource::delta) for whoever reads them first.
                const bool defer = lazy_ok && !douts.empty();
                if (st == NNVHIP_OK && !douts.empty()) {
                  double sums_only = 0.0;  // what the pass then writes: centre columns and partial sums
                  for (const DeltaOut& d : douts) sums_only += 8.0 * (double)Mp + 32.0 * (double)ldo * (double)delta_tile_chunks(d.ncols);
                  BufRef sums_at;
                  st = launch_delta_tiles(c, Wd, Mp, Mp, bias, ldo, (int64_t)douts.size(), douts.data(), dgroup.data(), max_cols,
                                          defer ? sums_only : dbytes, !defer, &sums_at);
                  for (size_t k = 0; k < dset.size() && st == NNVHIP_OK && sums_at; ++k) {
                    nnvhip_star* o = outs[dset[k]];
                    o->rng_at_buf = sums_at;
                    o->rng_part_at = sums_at->as<const double*>() + k;
                    o->rng_chunks_at = tiles_of[dset[k]];
                  }
                }
                if (st == NNVHIP_OK && defer) {
                  Ref<DeltaCall> call = make_ref<DeltaCall>();
                  call->W = fc->W;
                  call->bias = fc->bias;
                  call->base = basebuf;
                  call->S = shared_rows;
                  call->cprod = cprod;
                  call->lists = delta;
                  call->arena = outs[0]->Vbuf;
                  call->A = Wd;
                  call->bias_ptr = bias;
                  call->lda = Mp;
                  call->Mp = Mp;
                  call->ldo = ldo;
                  call->max_cols = max_cols;
                  call->bytes = dbytes;
                  call->outs = douts;
                  for (DeltaOut& d : call->outs) d.rpart = nullptr;
                  call->group = dgroup;
                  for (int64_t a = 0; a < nact; ++a) {
                    nnvhip_star* o = outs[act[(size_t)a]];
                    o->cs.delta = call;
                    if (c->poison_pending && dense[act[(size_t)a]] > 1 &&  // debugging aid: NaNs where nothing was written
                        hipMemsetAsync(o->V + o->ld, 0xff, sizeof(double) * o->ld * (dense[act[(size_t)a]] - 1), c->stream) != hipSuccess)
                      st = NNVHIP_ERR_HIP;
                  }
                }
                delta_done = true;
                bias_in_kernel = true;
              }
            }
          }
          auto nfull_of = [&](int64_t i) { return shared ? shapes[(size_t)shape_of[i]].nfull : 0; };
          int64_t total = 0;
          if (!delta_done) {
          for (int64_t i = 0; i < count; ++i)
            if (!filled[i]) {
              if (shared) {  // the columns past the last whole tile only, in a tile of their own width
                const int64_t rem = dense[i] - 128 * nfull_of(i);
                ldt[i] = rem > 64 ? 128 : rem > 32 ? 64 : rem > 0 ? 32 : 0;
              } else {
                ldt[i] = round_up(dense[i], 128);
              }
              total += kps[i] * ldt[i];
            }
          if (total > 0 && st == NNVHIP_OK) st = c->alloc(sizeof(double) * total, &packed);
          int64_t pos = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
            if (!filled[i] && ldt[i] > 0) {
              bt[i] = packed->as<double>() + pos;
              PackSet ps = pack_of(in[i], rws[i].kmap, packed->as<double>() + pos, kps[i], dense[i]);
              ps.ldt = ldt[i];
              if (shared) {
                ps.col0 = (int32_t)(128 * nfull_of(i));
                ps.ncols = (int32_t)(dense[i] - 128 * nfull_of(i));
              }
              packs.push_back(ps);
              pos += kps[i] * ldt[i];
            }
          if (st == NNVHIP_OK && !packs.empty()) st = launch_pack_rows_t(c, (int64_t)packs.size(), packs.data());
          for (int64_t i = 0; i < count; ++i) {
            tiles_of[i] = filled[i] ? 0 : ceil_div(dense[i], 128);
            chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
          }
          if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
          // tiles by width: [0] 128 columns, [1] 64, [2] 32 (the last tile of a set whose remainder fits); [3]: the
          // 128-column tiles that gather their rows of B from the shared matrix
          std::vector<SegTile> tiles[4];
          double flop[4] = {0.0, 0.0, 0.0, 0.0};
          int64_t off = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
            for (int64_t j = 0; j < dense[i] && !filled[i]; j += 128) {
              const int64_t valid = std::min<int64_t>(128, dense[i] - j);
              const bool gather = shared && j < 128 * nfull_of(i);
              const int w = gather ? 3 : valid > 64 ? 0 : valid > 32 ? 1 : 2;
              SegTile sg{};
              sg.kmap = rws[i].kmap;
              if (gather) {
                const RowShape& r = shapes[(size_t)shape_of[i]];
                sg.Bt = shared_rows->as<double>() + r.off;
                sg.ldbt = r.ldws;
                sg.b_col0 = j;
                sg.centre = in[i]->V;
                sg.gather_b = 1;
                sg.zero_row = (int32_t)r.rows;
              } else {
                sg.Bt = bt[i];
                sg.ldbt = ldt[i];
                sg.b_col0 = shared ? 0 : j;
              }
              sg.col_local0 = j;
              sg.col_base = off + j;
              sg.kp = (int32_t)kps[i];
              sg.valid = (int32_t)valid;
              sg.plb = outs[i]->plb;
              sg.pub = outs[i]->pub;
              sg.rpart = sums->as<double>() + 4 * ldo * (chunk_off[i] + j / 128);
              tiles[w].push_back(sg);
              flop[w] += 2.0 * (double)fc->Mp * (double)kps[i] * (double)valid;
            }
            off += in[i]->n + 1;
          }
          static const int widths[4] = {128, 64, 32, 128};
          for (int w = 3; w >= 0 && st == NNVHIP_OK; --w) {
            if (tiles[w].empty()) continue;
            BufRef dt;
            st = c->upload_table(tiles[w].data(), sizeof(SegTile) * tiles[w].size(), &dt);
            if (st == NNVHIP_OK)
              st = launch_gemm_seg(c, Wd, fc->Mp, outs[0]->V, ldo, fc->Mp, bias, widths[w], dt->as<SegTile>(), (int64_t)tiles[w].size(),
                                   flop[w], w == 3);
          }
          bias_in_kernel = true;
          }  // !delta_done
        } else {
        // several row tiles would each gather the kept rows of B: pack them once per set instead
        BufRef packed;
        std::vector<PackSet> packs;
        std::vector<const double*> bk((size_t)count, nullptr);
        {
          int64_t total = 0;
          for (int64_t i = 0; i < count; ++i)
            if (pk[i]) total += kps[i] * dense[i];
          if (total > 0) st = c->alloc(sizeof(double) * total, &packed);
          int64_t pos = 0;
          for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
            if (pk[i]) {
              bk[i] = packed->as<double>() + pos;
              packs.push_back(pack_of(in[i], rws[i].kmap, packed->as<double>() + pos, kps[i], dense[i]));
              pos += kps[i] * dense[i];
            }
          if (st == NNVHIP_OK && !packs.empty()) st = launch_pack_rows(c, (int64_t)packs.size(), packs.data());
        }
        const int64_t ldo = outs[0]->ld;
        for (int64_t i = 0; i < count; ++i) {
          tiles_of[i] = filled[i] ? 0 : ceil_div(dense[i], tn);
          chunk_off[i + 1] = chunk_off[i] + tiles_of[i] + (gs[i].m > 0 ? gch_part : 0);
        }
        if (st == NNVHIP_OK && chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
        int64_t off = 0, off_in = 0, kp_max = kLdAlign;
        for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
          for (int64_t j = 0; j < dense[i] && !filled[i]; j += tn) {
            GemmSeg sg;
            sg.plb = outs[i]->plb;
            sg.pub = outs[i]->pub;
            sg.rpart = sums->as<double>() + 4 * ldo * (chunk_off[i] + j / tn);
            sg.kmap = rws[i].kmap;
            sg.Bk = bk[i];
            sg.ldbk = kps[i];
            sg.col_local0 = j;
            sg.b_col_base = off_in + j;
            sg.col_base = off + j;
            sg.kp = (int32_t)kps[i];
            sg.valid = (int32_t)std::min<int64_t>(tn, dense[i] - j);
            segs.push_back(sg);
          }
          if (!filled[i]) {
            rows.flop += 2.0 * (double)fc->Mp * (double)kps[i] * (double)dense[i];
            kp_max = std::max(kp_max, kps[i]);
          }
          off += in[i]->n + 1;
          off_in += in[i]->stored_cols();
        }
        BufRef dsegs;
        if (st == NNVHIP_OK && !segs.empty()) st = c->upload_table(segs.data(), sizeof(GemmSeg) * segs.size(), &dsegs);
        if (st == NNVHIP_OK && !segs.empty()) {
          rows.segs = dsegs->as<GemmSeg>();
          st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, tn * (int64_t)segs.size(),
                           kp_max, bias, nullptr, &rows);
        }
        }
      } else {
        st = launch_gemm(c, Wd, fc->Mp, in[0]->V, in[0]->ld, outs[0]->V, outs[0]->ld, fc->Mp, cols, fc->Kp, bias);
      }
      if (st == NNVHIP_OK && bias && count > 1 && !bias_in_kernel) {
        // the GEMM adds the bias to column 0 of the arena (the first set's centre); the other sets'
        // centres get it here (a set whose dense columns the gather pass fills has it from there)
        std::vector<double*> centres;
        for (int64_t i = 1; i < count; ++i)
          if (!filled[i]) centres.push_back(outs[i]->V);
        BufRef tab;
        if (!centres.empty()) st = c->upload_table(centres.data(), sizeof(double*) * centres.size(), &tab);
        if (st == NNVHIP_OK && !centres.empty()) st = launch_bias_columns(c, tab->as<double*>(), (int64_t)centres.size(), bias, fc->Mp);
      }
      if (st == NNVHIP_OK && (any_onehot || any_fill)) {
        // the gather also leaves the range sums of its columns on the output handles, so the ReLU
        // that follows scans only the contracted columns
        const int64_t ldo = outs[0]->ld;
        if (!sums) {  // no segmented GEMM ran: the gather's chunks are all there is
          for (int64_t i = 0; i < count; ++i) chunk_off[i + 1] = chunk_off[i] + (gs[i].m > 0 ? gch_part : 0);
          if (chunk_off[count] > 0) st = c->alloc(sizeof(double) * 4 * ldo * chunk_off[count], &sums);
        }
        if (st == NNVHIP_OK && use_mm) {
          if (mm_early) mm_sums = mm_early;  // queued at the start of the call, from the same lists
          else {
            bool zero = true;
            for (int64_t i = 0; i < count; ++i) zero = zero && (gs[i].m == 0 || in[i]->oh_plb_zero);
            st = launch_range_sums_mm(c, fc, count, gs.data(), &mm_sums, &mm_slot, zero);
          }
        }
        if (st == NNVHIP_OK) {
          for (int64_t i = 0; i < count; ++i) {
            gs[i].part = (gch_part > 0 && gs[i].m > 0) ? sums->as<double>() + 4 * ldo * (chunk_off[i] + tiles_of[i]) : nullptr;
            lazy[i] = lazy_ok && (gs[i].part != nullptr || (use_mm && gs[i].m > 0));
            gs[i].lazy = lazy[i];
          }
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, ldo, count, gs.data(), gch_part);
        }
      }
      // what the two passes left: the GEMM tiles' chunks cover the contracted columns, the gather's its own;
      // columns covered by neither (a GEMM without the fused sums) still need a scan, filled zeros add nothing
      for (int64_t i = 0; i < count && st == NNVHIP_OK && (sums || mm_sums); ++i) {
        const int64_t nchunks = chunk_off[i + 1] - chunk_off[i];
        const bool mm = mm_sums && gs[i].m > 0;
        if (nchunks == 0 && !mm) continue;
        if (nchunks > 0) {
          outs[i]->rng_buf = sums;
          outs[i]->rng_part = sums->as<double>() + 4 * outs[0]->ld * chunk_off[i];
          outs[i]->rng_chunks = nchunks;
        }
        if (mm) {
          outs[i]->rng_mm_buf = mm_sums;
          outs[i]->rng_mm = mm_sums->as<double>() + 4 * outs[0]->ld * mm_slot[(size_t)i];  // two columns of 2 * ld entries
        }
        outs[i]->rng_first_col = (filled[i] || tiles_of[i] > 0) ? 1 : dense[i];
      }
    } else {
      for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i) {
        GemmRows rows;
        int64_t kp = fc->Kp;
        bool pack = false;
        const bool compact = rows_of(i, &rows, &kp, &pack);
        if (compact && nothing_kept(i, rows)) {
          fill_by_gather(i);
          st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[i]->ld, 1, &gs[i], 0);
          continue;
        }
        BufRef packed;
        if (compact && pack) {
          st = c->alloc(sizeof(double) * kp * dense[i], &packed);
          if (st != NNVHIP_OK) break;
          PackSet ps = pack_of(in[i], in[i]->kept_idx, packed->as<double>(), kp, dense[i]);
          st = launch_pack_rows(c, 1, &ps);
          if (st != NNVHIP_OK) break;
          rows.Bk = packed->as<double>();
          rows.ldbk = kp;
        }
        st = launch_gemm(c, Wd, fc->Mp, in[i]->V, in[i]->ld, outs[i]->V, outs[i]->ld, fc->Mp, dense[i], kp, bias, nullptr,
                         compact ? &rows : nullptr);
        if (st == NNVHIP_OK && gs[i].m > 0) st = launch_gather_columns(c, Wd, fc->Mp, fc->Mp, outs[i]->ld, 1, &gs[i], 0);
      }
    }
    // the gathered columns remember where they came from
    // (arrays: the next layer packs kept rows of these columns, i.e. reads rows of W - from a row-major copy)
    if (st == NNVHIP_OK && count >= 64 && !fc->Wt && fc->Mp * fc->Kp < (int64_t(1) << 31)) {
      bool any = false;
      for (int64_t i = 0; i < count; ++i) any = any || gs[i].m > 0;
      if (any) {
        BufRef wt;
        st = c->alloc(sizeof(double) * fc->Mp * fc->Kp, &wt);
        if (st == NNVHIP_OK) {
          hipLaunchKernelGGL(transpose_weights_kernel, dim3((unsigned)ceil_div(fc->Kp, 32), (unsigned)ceil_div(fc->Mp, 32)), dim3(32, 8), 0,
                             c->stream, Wd, wt->as<double>(), (int)fc->Mp, (int)fc->Kp);
          if (hipGetLastError() != hipSuccess) st = NNVHIP_ERR_HIP;
          fc->Wt = wt;
        }
      }
    }
    for (int64_t i = 0; i < count && st == NNVHIP_OK; ++i)
      if (gs[i].m > 0) {
        nnvhip_star* o = outs[i];
        ColSource& cs = o->cs;
        cs.W_buf = fc->W;
        cs.W = Wd;
        cs.ldw = fc->Mp;
        cs.rows = fc->Mp;
        if (fc->Wt) {
          cs.Wt_buf = fc->Wt;
          cs.Wt = fc->Wt->as<double>();
          cs.ldwt = fc->Kp;
        }
        cs.idx_buf = in[i]->oh_idx_buf;
        cs.idx = gs[i].idx;
        cs.scale_buf = in[i]->oh_scale_buf;
        cs.scale = gs[i].scale;
        cs.from = dense[i];
        cs.cols = gs[i].m;
        cs.pending = lazy[i] != 0;
        cs.zero_to = (lazy[i] && gs[i].nfill > 0) ? gs[i].nfill : 0;  // a filled set's leading columns
        // debugging aid: NaNs where nothing was written, so that a reader that forgets to ask for the
        // columns cannot pass a test on what an earlier call happened to leave in the memory
        auto poison = [&](double* p, int64_t ncols) -> int {
          NNV_HIP_TRY(hipMemsetAsync(p, 0xff, sizeof(double) * o->ld * ncols, c->stream));
          return NNVHIP_OK;
        };
        if (c->poison_pending && cs.pending) st = poison(o->V + cs.from * o->ld, cs.cols);
        if (c->poison_pending && cs.zero_to > 1 && st == NNVHIP_OK) st = poison(o->V + o->ld, cs.zero_to - 1);
      }
  }
  if (st == NNVHIP_OK) st = c->end_op();
  if (st != NNVHIP_OK) {
    release_all(outs);
    return st;
  }
  for (int64_t i = 0; i < count; ++i) out[i] = outs[i];
  return NNVHIP_OK;
}

}  // extern "C"
