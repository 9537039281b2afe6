// Host-side bounds check of the direct-to-LDS kernels (build with -DMI_HOST_CHECK, `make host-check`).
//
// The fast kernel (gemm_fast.hpp) has no bounds checks of its own: whether a launch stays inside its operands is
// decided by the host code that picks tiles, grids and variants.  In this build no kernel is launched.  Instead every
// launch of the fast kernel lands in fast_launch() below, which walks the grid -- every workgroup, wavefront and lane
// -- through the same integer functions the device code uses for its addresses (workgroup -> tile, the loaders'
// lane offsets and K-tile stepping, addend and epilogue geometry, accumulator images, partial-sum slots; all marked
// MI_HD in gemm_fast.hpp) and checks that every byte a lane would read or write lies inside a buffer the caller
// registered, and that every tile of the product is computed exactly once.  The host code that leads to the launch
// (argument validation, workspace layout, cost model, step grouping, launchers) is the library's own, compiled with
// AddressSanitizer and UndefinedBehaviorSanitizer.
//
// What is replayed by hand here, because it is control flow and not address arithmetic: which K tiles a workgroup
// requests (all of [0, nk): the guards of the prologue and of the steady and tail loops), and which epilogue a variant
// runs.
//
// The other kernels (normalisation passes, transposes, the general tile kernel, the per-head kernels) guard their own
// accesses or run on exact multiples of their slices; what can go wrong for them is the host side: a workspace segment
// carved too small, a stride or a count passed wrongly.  Their launch sites state, with MI_FOOTPRINT (launch.hpp), the
// block of memory every pointer argument of the launch covers, and footprint() below checks each block against the
// registered buffers the same way.
#pragma once
#include <cstdint>
#include <cstdio>
#include <map>
#include <tuple>
#include <vector>

#include "gemm_fast.hpp"

namespace mi {
namespace host_check {

struct Range {
  uint64_t lo, hi;
  const char* name;
};
struct State {
  std::vector<Range> ranges;
  long launches = 0, workgroups = 0, accesses = 0, failures = 0;
  long other_launches = 0, footprints = 0;  // launches of the self-guarding kernels, blocks of memory they stated
  const char* context = "";
  bool exhaustive = false;  // walk the lanes of every workgroup and every K tile instead of the sample described below
  uint64_t hit_lo = 1, hit_hi = 0;  // the buffer the last access fell into (consecutive accesses mostly share one)
};
inline State g_state;
inline State& state() { return g_state; }

inline void add_range(const void* p, size_t bytes, const char* name) {
  if (p != nullptr && bytes > 0) state().ranges.push_back(Range{(uint64_t)(uintptr_t)p, (uint64_t)(uintptr_t)p + bytes, name});
}
inline void clear_ranges() {
  state().ranges.clear();
  state().hit_lo = 1;
  state().hit_hi = 0;
}

inline void report(const char* what, uint64_t addr, size_t bytes, const char* detail) {
  State& st = state();
  if (++st.failures <= 20) {
    std::fprintf(stderr, "[host-check] %s: %s of %zu bytes at %#llx is outside every registered buffer (%s)\n", st.context, what, bytes,
                 (unsigned long long)addr, detail);
    for (const Range& r : st.ranges)
      std::fprintf(stderr, "    %-12s [%#llx, %#llx)\n", r.name, (unsigned long long)r.lo, (unsigned long long)r.hi);
  }
}
inline void fail(const char* msg) {
  State& st = state();
  if (++st.failures <= 20) std::fprintf(stderr, "[host-check] %s: %s\n", st.context, msg);
}

// The access must lie wholly inside one registered buffer.  (Called billions of times: the checker's own bookkeeping is
// left out of the sanitizers' instrumentation, the library's code is not.)
__attribute__((no_sanitize("address", "undefined"))) inline void touch(uint64_t addr, size_t bytes, const char* what,
                                                                         const char* detail = "") {
  State& st = g_state;
  ++st.accesses;
  if (addr >= st.hit_lo && addr + bytes <= st.hit_hi) return;
  for (const Range& r : st.ranges)
    if (addr >= r.lo && addr + bytes <= r.hi) {
      st.hit_lo = r.lo;
      st.hit_hi = r.hi;
      return;
    }
  report(what, addr, bytes, detail);
}
template <class T>
inline void touch(const T* p, size_t bytes, const char* what, const char* detail = "") {
  touch((uint64_t)(uintptr_t)p, bytes, what, detail);
}

// One pointer argument of a self-guarding kernel: `batch` blocks `batch_stride` elements apart, each of `rows` rows of
// `cols` elements that start `ld` elements apart, `elem` bytes per element.  Every block must lie inside one registered
// buffer (all blocks of up to 4096 batch entries, the two ends beyond that: the blocks are equally spaced).
inline void footprint(const char* what, const void* base, size_t elem, int64_t batch, int64_t batch_stride, int64_t rows, int64_t ld,
                      int64_t cols) {
  if (base == nullptr || batch <= 0 || rows <= 0 || cols <= 0) return;
  State& st = state();
  ++st.footprints;
  if (batch_stride < 0 || ld < cols) fail("a footprint with rows that overlap");
  const size_t bytes = (size_t)((rows - 1) * ld + cols) * elem;
  const char* b0 = static_cast<const char*>(base);
  for (int64_t b = 0; b < batch; ++b) {
    if (batch > 4096 && b == 1) b = batch - 1;
    touch(b0 + (size_t)b * batch_stride * elem, bytes, what, "whole block of a self-guarding kernel");
  }
}
inline void other_launch() { ++state().other_launches; }

// The scalars every tile kernel resolves per batch entry (resolve_shift in gemm_engine.hpp) and the partial sums its
// workgroups leave: `slots` workgroups per batch entry write one float each.
inline void scalar_footprints(const GemmParams& p, int64_t batch, int64_t slots) {
  if (p.shift_mode == SHIFT_GRAM) {
    footprint("partial sums read", p.slots_in, sizeof(float), batch, p.nslots_in, 1, p.nslots_in, p.nslots_in);
    footprint("shift written", p.shift_io, sizeof(float), 1, 0, 1, batch, batch);
  } else if (p.shift_mode != SHIFT_NONE) {
    footprint("shift read", p.shift_io, sizeof(float), 1, 0, 1, batch, batch);
  }
  footprint("input scale read", p.xscale, sizeof(float), 1, 0, 1, batch, batch);
  if (p.slots_out != nullptr) footprint("partial sums written", p.slots_out + p.slot_base, sizeof(float), batch, p.slot_stride, 1, slots, slots);
}

// A launch of the general tile kernel (gemm_engine.hpp; every access guarded by the matrix extents): operands, addends
// and result as the extents in `p` describe them.
inline void general_launch(const GemmParams& p, int64_t batch, bool p_ks, bool q_ks, bool syrk, bool out_f32, int64_t tiles) {
  other_launch();
  const int64_t inner = p.batch_inner > 1 ? p.batch_inner : 1, outer = batch / inner;
  if (batch % inner != 0) fail("batch is not a whole number of inner batches");
  for (int64_t in = 0; in < inner; ++in) {
    const int64_t p2 = p.batch_inner > 1 ? in * p.p_bs2 : 0, q2 = p.batch_inner > 1 ? in * p.q_bs2 : 0;
    footprint("operand P", p.P + p2, 2, outer, p.p_bs, p_ks ? p.K : p.M, p.ldp, p_ks ? p.M : p.K);
    footprint("operand Q", p.Q + q2, 2, outer, p.q_bs, q_ks ? p.K : p.N, p.ldq, q_ks ? p.N : p.K);
  }
  // (the addends are read whenever their pointers are given: the coefficients are resolved on the device)
  footprint("addend", p.Cin, 2, batch, p.c_bs, p.M, p.ldc, p.N);
  footprint("second addend", p.Cin2, 2, batch, p.c_bs, p.M, p.ldc, p.N);
  footprint("result", p.Out, out_f32 ? 4 : 2, batch, p.o_bs, p.M, p.ldo, p.N);
  scalar_footprints(p, batch, syrk ? 0 : tiles);
}

template <class C, bool P_KS, bool Q_KS, int MODE, bool OUT_F32, bool EDGE, int STREAMK, bool RMW>
void fast_launch(dim3 grid, const GemmParams& p) {
  State& st = state();
  ++st.launches;
  constexpr int NS = C::NS, FM = C::FM, FN = C::FN, NT = C::NT, MI = C::MI;
  constexpr bool SYRK_STAGED = MODE == MODE_SYRK && !OUT_F32 && C::NW == 4;
  constexpr bool GEMM_STAGED = MODE == MODE_GEMM && (C::TN == 32 || C::TN == 64 || C::TN == 128);
  constexpr bool CIN_EARLY = SYRK_STAGED && SyrkStage<C>::CIN_EARLY;
  static_assert(SYRK_STAGED || GEMM_STAGED, "every instance of the fast kernel runs one of the two staged epilogues");
  static_assert(!(EDGE && (P_KS || Q_KS)), "no edge variant for K-strided operands");
  (void)NS;
  const int esz = OUT_F32 ? 4 : 2;
  // (batch entry, tile row, tile column) -> K tiles computed, to check that every tile is computed exactly once
  std::map<std::tuple<int64_t, int, int>, int> covered;
  const int nk_full = p.K / C::BK;
  if (p.K % C::BK != 0 || nk_full < 1) fail("K is not a whole number of K tiles");

  // Every workgroup is decoded (tile coverage); the lanes of all workgroups are walked for grids of up to 640
  // workgroups, of the first and last 128 and of every (total / 256)-th one for larger grids (addresses are affine in
  // the tile indices between the ends).  `exhaustive` drops both samples: every workgroup, every K tile.
  const long total = (long)grid.x * (long)grid.y;
  const long every = total > 640 ? total / 256 : 1;
  for (unsigned by = 0; by < grid.y; ++by) {
    for (unsigned bx = 0; bx < grid.x; ++bx) {
      const long index = (long)by * grid.x + bx;
      const bool walk_lanes = st.exhaustive || total <= 640 || index < 128 || index >= total - 128 || index % every == 0;
      const int bid = (int)bx;
      int64_t batch = by;
      int tm, tn, k_first = 0, nk = nk_full, sk_tile = 0, sk_split = 0;
      if constexpr (MODE == MODE_SYRK) {
        const int tri = p.tiles_m * (p.tiles_m + 1) / 2;
        int tile;
        if constexpr (STREAMK == SK_NONE) {
          tile = tri_tile_of_block(bid, p.lin_tiles, p.lin_g);
          if (tile < 0) continue;
          if (tile >= p.lin_tiles) fail("tile number beyond the launch");
        } else {
          if constexpr (STREAMK == SK_PARTS) {
            if (!sk_part_of_block(bid, p.sk_tpx, p.sk_rem, p.sk_splits, nk_full, sk_tile, sk_split, k_first, nk)) continue;
            if (k_first < 0 || nk < 1 || k_first + nk > nk_full) fail("K range of a split outside the operand");
          } else {
            if (!sk_quarter_of_block(bid, p.sk_rem, sk_tile, sk_split)) continue;
          }
          tile = p.lin_tiles + sk_tile;
        }
        batch = tile / tri;
        tri_block_decode(tile % tri, p.tiles_m, tm, tn);
        if (tn > tm || tm >= p.tiles_m) fail("tile outside the lower triangle");
        if constexpr (STREAMK == SK_FINISH) {
          const int qm = sk_split % 2, qn = sk_split / 2;
          if (tm == tn && qn > qm) continue;
          tm = 2 * tm + qm;
          tn = 2 * tn + qn;
        }
      } else {
        gemm_tile_of(bid, p.tiles_m, p.tiles_n, tm, tn);
        if (tm < 0 || tm >= p.tiles_m || tn < 0 || tn >= p.tiles_n) fail("GEMM tile outside the grid");
      }
      covered[std::make_tuple(batch, tm, tn)] += (STREAMK == SK_FINISH) ? nk_full : nk;
      const int m0 = tm * C::TILE_M, n0 = tn * C::TILE_N;
      int64_t p_off = batch * p.p_bs, q_off = batch * p.q_bs;
      if (p.batch_inner > 1) {
        const int64_t outer = batch / p.batch_inner, inner = batch % p.batch_inner;
        p_off = outer * p.p_bs + inner * p.p_bs2;
        q_off = outer * p.q_bs + inner * p.q_bs2;
      }
      const bool diag = MODE == MODE_SYRK && tm == tn;
      if (!walk_lanes) continue;
      ++st.workgroups;
      // scalars (resolve_shift): partial sums, the shift and the input scale of this batch entry
      if (p.shift_mode == SHIFT_GRAM) {
        if (p.nslots_in > 0) touch(p.slots_in + batch * p.nslots_in, sizeof(float) * (size_t)p.nslots_in, "partial sums read");
        touch(p.shift_io + batch, sizeof(float), "shift written");
      } else if (p.shift_mode != SHIFT_NONE) {
        touch(p.shift_io + batch, sizeof(float), "shift read");
      }
      if (p.xscale != nullptr) touch(p.xscale + batch, sizeof(float), "input scale read");
      if (MODE == MODE_GEMM && GEMM_STAGED && p.slots_out != nullptr)
        touch(p.slots_out + batch * p.slot_stride + p.slot_base + bid, sizeof(float), "partial sum written");

      for (int wave = 0; wave < C::NW; ++wave) {
        const int wm = wave % C::WGM, wn = wave / C::WGM;
        const bool idle_wave = (m0 + wm * C::TM >= p.M) || (n0 + wn * C::TN >= p.N) ||
                               (MODE == MODE_SYRK && tm == tn && wn * C::TN >= (wm + 1) * C::TM);
        for (int lane = 0; lane < 64; ++lane) {
          const int tid = wave * 64 + lane;
          // ---- operand tiles: every wavefront, idle or not, requests its share of K tiles [0, nk)
          if constexpr (STREAMK != SK_FINISH) {
            FastLoader<C, P_KS, C::TILE_M, EDGE> lp;
            FastLoader<C, Q_KS, C::TILE_N, EDGE> lq;
            lp.init(p.P + p_off + (STREAMK ? (int64_t)k_first * C::BK : 0), p.ldp, m0, p.M, wave, lane);
            lq.init(p.Q + q_off + (STREAMK ? (int64_t)k_first * C::BK : 0), p.ldq, n0, p.N, wave, lane);
            for (int kt = 0; kt < nk; ++kt) {
              if (kt < 2 || kt >= nk - 2 || st.exhaustive) {  // (the address of a load is affine in kt: the ends bound the rest)
                for (int i = 0; i < decltype(lp)::LPT; ++i) touch(lp.address(i), 16, "operand P load");
                for (int i = 0; i < decltype(lq)::LPT; ++i) touch(lq.address(i), 16, "operand Q load");
              }
              lp.advance();
              lq.advance();
            }
          }
          // ---- first addend in accumulator layout, requested in front of the K loop
          if constexpr (CIN_EARLY) {
            if (p.Cin != nullptr)
              for (int i = 0; i < FM; ++i)
                for (int j = 0; j < FN; ++j)
                  touch(p.Cin + batch * p.c_bs + syrk_addend_elem<C, EDGE>(p.M, p.N, p.ldc, lane, m0 + wm * C::TM, n0 + wn * C::TN, i, j), 8,
                        "first addend");
          }
          if constexpr (STREAMK == SK_PARTS) {
            if (!idle_wave)
              for (int i = 0; i < FM; ++i)
                for (int j = 0; j < FN; ++j)
                  touch(reinterpret_cast<const char*>(p.sk_partials) + 16 * sk_image_quad(sk_split, p.sk_rem, sk_tile, i, j, tid), 16,
                        "accumulator image written");
            continue;
          }
          if constexpr (STREAMK == SK_FINISH) {
            if (!idle_wave)
              for (int s = 0; s < p.sk_splits; ++s)
                for (int i = 0; i < FM; ++i)
                  for (int j = 0; j < FN; ++j)
                    touch(reinterpret_cast<const char*>(p.sk_partials) +
                              16 * sk_image_quad(s, p.sk_rem, sk_tile, wm * FM + i, wn * FN + j, sk_split * 64 + lane),
                          16, "accumulator image read");
          }
          // ---- epilogue
          if constexpr (GEMM_STAGED && MODE == MODE_GEMM) {
            using G = GemmStage<C>;
            const int m_base = m0 + wm * C::TM, n_base = n0 + wn * C::TN;
            const bool use_c = p.beta != 0.0f && p.Cin != nullptr;
            const char* out = static_cast<const char*>(p.Out) + batch * p.o_bs * esz;
            for (int i = 0; i < FM; ++i) {
              for (int t = 0; t < G::NIT; ++t) {
                int dm, dn;
                G::piece_of(lane, i, t, dm, dn);
                const int m = m_base + dm, n = n_base + dn;
                const bool inside = !EDGE || (m < p.M && n < p.N);
                if (use_c && inside) touch(p.Cin + batch * p.c_bs + (int64_t)m * p.ldc + n, 16, "GEMM addend");
                if (!inside) continue;
                if (!(OUT_F32 && !EDGE && p.out_transposed)) touch(out + ((int64_t)m * p.ldo + n) * esz, 8 * (size_t)esz, "GEMM result");
              }
              if (OUT_F32 && !EDGE && p.out_transposed) {
                for (int t = 0; t < C::TN / 16; ++t) {
                  int dm, dn;
                  G::transposed_piece_of(lane, i, t, dm, dn);
                  touch(out + ((int64_t)(n_base + dn) * p.ldo + m_base + dm) * 4, 16, "GEMM result, transposed");
                }
              }
            }
          }
          if constexpr (SYRK_STAGED) {
            using S = SyrkStage<C>;
            const uint16_t* ob = static_cast<const uint16_t*>(p.Out) + batch * p.o_bs;
            const uint16_t* Cb = p.Cin ? p.Cin + batch * p.c_bs : nullptr;
            const uint16_t* Cb2 = p.Cin2 ? p.Cin2 + batch * p.c_bs : nullptr;
            // (the addends are read whenever their pointers are given: the coefficients are resolved on the device)
            if constexpr (S::CIN_EARLY) {
              if (Cb2 != nullptr)
                for (int i = 0; i < FM; ++i)
                  for (int j = 0; j < FN; ++j)
                    touch(Cb2 + syrk_addend_elem<C, EDGE>(p.M, p.N, p.ldc, lane, m0 + wm * C::TM, n0 + wn * C::TN, i, j), 8, "second addend");
            } else {
              for (const uint16_t* src : {Cb, Cb2}) {
                if (src == nullptr) continue;
                for (int u = 0; u < S::NCH; ++u) {
                  int row, c8;
                  S::chunk_of(tid, u, row, c8);
                  const int gr = m0 + row, gc = n0 + c8 * 8;
                  if (!EDGE || (gr < p.M && gc < p.N)) touch(src + (int64_t)gr * p.ldc + gc, 16, "addend copied to the staging area");
                }
              }
            }
            for (int it = 0; it < S::NCH; ++it) {
              int row, c8;
              S::chunk_of(tid, it, row, c8);
              const int gr = m0 + row, gc = n0 + c8 * 8;
              if (S::chunk_held(diag, row, c8) && (!EDGE || (gr < p.M && gc < p.N))) touch(ob + (int64_t)gr * p.ldo + gc, 16, "tile written");
            }
            if (!p.skip_upper) {
              auto mirror = [&](auto rows_c, auto ccols_c, int r_lo, int grow0, int gcol0) {
                constexpr int ROWS = decltype(rows_c)::value, CCOLS = decltype(ccols_c)::value;
                for (int it = 0; it < S::template mirror_iterations<ROWS, CCOLS>(); ++it) {
                  int src_row, src_col, drow, dcol;
                  const bool on = S::template mirror_piece<ROWS, CCOLS>(it, wave, lane, r_lo, src_row, src_col, drow, dcol);
                  // (two transpose reads: four columns at src_row and at src_row + 4)
                  if (src_row < 0 || src_row + 4 >= S::TILE || src_col < 0 || src_col + 3 >= S::TILE) fail("mirror read outside the staged tile");
                  const int gr = grow0 + drow, gc = gcol0 + dcol;
                  if (on && (!EDGE || (gr < p.N && gc < p.M))) touch(ob + (int64_t)gr * p.ldo + gc, 16, "mirror image written");
                }
              };
              if (!diag)
                mirror(std::integral_constant<int, S::TILE>{}, std::integral_constant<int, S::TILE>{}, 0, n0, m0);
              else
                mirror(std::integral_constant<int, C::TM>{}, std::integral_constant<int, C::TM>{}, C::TM, n0, m0 + C::TM);
            }
          }
        }
      }
    }
  }
  // every tile of the launch exactly once, over its whole K range
  if constexpr (STREAMK == SK_NONE || STREAMK == SK_FINISH) {
    for (const auto& kv : covered)
      if (kv.second != nk_full) fail("a tile is computed more than once");
    if constexpr (MODE == MODE_SYRK && STREAMK == SK_NONE) {
      if ((long)covered.size() != (long)p.lin_tiles) fail("the launch does not cover its tiles");
    } else if constexpr (MODE == MODE_GEMM) {
      if ((long)covered.size() != (long)p.tiles_m * p.tiles_n * (long)grid.y) fail("the launch does not cover its tiles");
    }
  } else {
    for (const auto& kv : covered)
      if (kv.second != nk_full) fail("the splits of a left-over tile do not add up to its K range");
    if ((long)covered.size() != (long)p.sk_rem) fail("the split launch does not cover the left-over tiles");
  }
}

}  // namespace host_check
}  // namespace mi
