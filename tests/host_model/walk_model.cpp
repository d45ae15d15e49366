// Host model of the walks the GPU kernels perform - test infrastructure, CPU only.
//
// The kernels of tritonops_amd/csrc keep several protocols by hand: which work
// item a persistent workgroup takes next, which LDS stage a KV tile lives in,
// how many vector-memory operations a counted wait leaves in flight, which
// blocks a window pair stands for.  This program restates those walks in plain
// C++ - no device code, no arithmetic of the attention itself except the
// running-reference softmax - and checks their invariants over thousands of
// shapes; it is built with -fsanitize=address,undefined by
// tests/test_host_model.py, so that an index that leaves its array fails loudly.
//
//   dense forward (prefill.hip, dense_kernel and its short form
//     dense_short_kernel): work-item map and persistent
//     schedule visit every (sequence, head, q tile) once; every LDS stage a wave
//     reads holds the tile it expects, requested, landed (the wave's counted
//     wait covers its loads) and published by a barrier; no stage is written in
//     a barrier interval in which a wave reads it; the Q registers have landed
//     before their first use.
//   block-sparse forward (prefill.hip, sparse_kernel): the two-stage K ring that
//     runs one tile ahead of the two-stage V ring; the block list held in two
//     64-entry registers; every tile read is the tile of the listed block.
//   softmax with a running reference point (no row maximum in the common
//     path): equals the plain softmax, also for scores that keep growing.
//   decode (decode.hip): the window form's arithmetic block list equals the
//     set of blocks that hold an attended token; live chunks are dealt once.
//   window walk (prefill.hip, dense_short_kernel with WIN): the tiles an item
//     of the two-window form walks, the positions each wave works on and the
//     tile masks let every query see exactly the keys the window rule allows.
#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <deque>
#include <random>
#include <set>
#include <string>
#include <vector>

static int g_fail = 0;
// 0: the kernels' protocols as they are.  1..12: one deliberate mistake each; the
// run must then fail (tests/test_host_model.py checks that it does), which is
// what shows that the checks below can tell a broken protocol from a sound one.
static int g_mut = 0;
#define CHECK(cond, ...)                                   \
  do {                                                     \
    if (!(cond)) {                                         \
      std::printf("FAIL %s:%d: ", __FILE__, __LINE__);     \
      std::printf(__VA_ARGS__);                            \
      std::printf("\n");                                   \
      if (++g_fail > 20) std::exit(1);                     \
    }                                                      \
  } while (0)

// ------------------------------------------------------------------ dense
namespace dense {
constexpr int NW = 8, NS = 4, TN = 64, BM = 256;

struct Shape {
  int batch, hq, hkv;
  std::vector<int> lens;  // per sequence (packed) - for the batched form all equal
  int max_seqlen;
  bool causal;
};

struct Geo {
  int b, kvh, h, qt, len;
};

// prefill.hip: item_geo
static bool item_geo(const Shape& s, int n_qtiles, int bid, Geo& g, int bm = BM) {
  const int gqa = s.hq / s.hkv;
  const int per_unit = n_qtiles * gqa;
  const int n_units = s.batch * s.hkv;
  int unit, r;
  if ((n_units & 7) == 0) {
    const int xcd = bid & 7, slot = bid >> 3;
    unit = (slot / per_unit) * 8 + xcd;
    r = slot % per_unit;
  } else {
    unit = bid / per_unit;
    r = bid % per_unit;
  }
  g.qt = n_qtiles - 1 - r / gqa;
  g.b = unit / s.hkv;
  g.kvh = unit % s.hkv;
  g.h = g.kvh * gqa + r % gqa;
  g.len = std::min(s.lens[g.b], s.max_seqlen);
  return g.qt * bm < g.len;
}

// One vector-memory operation of a wave, in issue order.
struct VmOp {
  enum Kind { Q, TILE, STORE } kind;
  int item, tile;  // TILE: which tile of which item
};

template <int NWAVES>
struct StageT {
  int item = -1, tile = -1;   // latest request
  int issued_in = -1;         // barrier interval of the latest request
  bool landed[NWAVES] = {};   // wave w's loads of it have retired
  bool published = false;     // a barrier has passed since all of them landed
};

struct Wave {
  std::deque<VmOp> vm;
  bool q_landed = false;
  int q_item = -1;
};

template <int NWAVES, int NSTAGES>
struct MachineT {
  using Stage = StageT<NWAVES>;
  Stage st[NSTAGES];
  Wave wv[NWAVES];
  int interval = 0;                 // barriers passed so far
  std::vector<std::pair<int, int>> reads_this_interval;  // (stage, wave)
  int ipw2;                         // loads per tile and wave (K + V)

  void retire(int w, const VmOp& op) {
    if (op.kind == VmOp::Q) {
      if (op.item == wv[w].q_item) wv[w].q_landed = true;
    } else if (op.kind == VmOp::TILE) {
      for (auto& s : st)
        if (s.item == op.item && s.tile == op.tile) s.landed[w] = true;
    }
  }
  void wait(int w, int n) {
    while ((int)wv[w].vm.size() > n) {
      retire(w, wv[w].vm.front());
      wv[w].vm.pop_front();
    }
  }
  void request_tile(int w, int stage, int item, int tile) {
    Stage& s = st[stage];
    if (s.item != item || s.tile != tile) {  // first wave to ask for it in this round
      s.item = item;
      s.tile = tile;
      s.issued_in = interval;
      s.published = false;
      for (bool& l : s.landed) l = false;
    }
    CHECK(s.issued_in == interval, "waves request tile %d of item %d in different barrier intervals", tile, item);
    for (int i = 0; i < ipw2; ++i) wv[w].vm.push_back({VmOp::TILE, item, tile});
    // nobody may read this stage in the interval in which it is being filled
    for (auto& r : reads_this_interval)
      CHECK(r.first != stage, "stage %d is requested in an interval in which wave %d reads it", stage, r.second);
  }
  void read(int w, int stage, int item, int tile, const char* what) {
    const Stage& s = st[stage];
    CHECK(s.item == item && s.tile == tile, "wave %d reads %s of tile %d (item %d) from stage %d, which holds tile %d (item %d)",
          w, what, tile, item, stage, s.tile, s.item);
    CHECK(s.published, "wave %d reads %s of tile %d (item %d) from stage %d before a barrier has published it", w, what,
          tile, item, stage);
    CHECK(s.issued_in < interval, "stage %d is read in the interval in which it was requested", stage);
    reads_this_interval.push_back({stage, w});
  }
  // every wave has arrived
  void barrier() {
    ++interval;
    reads_this_interval.clear();
    for (auto& s : st) {
      bool all = s.item >= 0;
      for (bool l : s.landed) all = all && l;
      if (all) s.published = true;
    }
  }
};

using Machine = MachineT<NW, NS>;

struct Item {
  int id, len, q0, n_tiles;
};

// The per-wave programs are run "barrier interval by barrier interval": inside
// an interval the waves are independent, so the model runs wave 0..7 one after
// the other up to their next barrier.  A program is a list of steps.
struct Step {
  enum Kind { WAIT, BARRIER, REQ_Q, REQ_TILE, READ, USE_Q, STORE, STAGE_TOUCH } kind;
  int a = 0, b = 0, c = 0;  // WAIT: n; REQ_TILE: stage, item, tile; READ: stage, item, tile; STORE: count
  const char* what = "";
};

// Runs the per-wave programs barrier interval by barrier interval: inside an
// interval the waves are independent, so wave 0, 1, ... each run up to their
// next barrier, then the barrier happens for all of them.
template <class M>
static void execute(std::vector<std::vector<Step>>& prog, M& m, int ksteps) {
  const int nw = (int)prog.size();
  std::vector<size_t> pc(nw, 0);
  for (;;) {
    int at_barrier = 0, done = 0;
    for (int w = 0; w < nw; ++w) {
      auto& P = prog[w];
      while (pc[w] < P.size() && P[pc[w]].kind != Step::BARRIER) {
        const Step& st = P[pc[w]++];
        switch (st.kind) {
          case Step::WAIT: m.wait(w, st.a); break;
          case Step::REQ_Q:
            m.wv[w].q_item = st.a;
            m.wv[w].q_landed = false;
            for (int i = 0; i < ksteps; ++i) m.wv[w].vm.push_back({VmOp::Q, st.a, 0});
            break;
          case Step::USE_Q:
            CHECK(m.wv[w].q_item == st.a && m.wv[w].q_landed, "wave %d uses the Q registers of item %d before its loads have retired", w, st.a);
            break;
          case Step::REQ_TILE: m.request_tile(w, st.a, st.b, st.c); break;
          case Step::READ: m.read(w, st.a, st.b, st.c, st.what); break;
          case Step::STORE:
            for (int i = 0; i < st.a; ++i) m.wv[w].vm.push_back({VmOp::STORE, 0, 0});
            break;
          case Step::STAGE_TOUCH:
            // the staging area must not be the target of a tile load that is under way
            CHECK(m.st[st.a].issued_in < m.interval || m.st[st.a].item < 0, "write-out stages through stage %d while a tile is being loaded into it", st.a);
            m.reads_this_interval.push_back({st.a, w});
            break;
          default: break;
        }
      }
      if (pc[w] < P.size()) ++at_barrier; else ++done;
    }
    if (done == nw) break;
    CHECK(at_barrier == nw, "waves disagree on the number of barriers (%d at a barrier, %d finished)", at_barrier, done);
    if (at_barrier != nw) break;
    for (int w = 0; w < nw; ++w) ++pc[w];
    m.barrier();
  }
}

static void run(const Shape& s, int grid, int ksteps, int ipw, int out_stores_full, Machine& m,
                std::vector<int>& visited) {
  const int n_qtiles = (s.max_seqlen + BM - 1) / BM;
  const int n_items = n_qtiles * s.hq * s.batch;
  m.ipw2 = 2 * ipw;
  for (int wg = 0; wg < grid; ++wg) {
    // ---- the items of this workgroup, as next_item() finds them
    std::vector<Item> items;
    int round = 0;
    for (int base = 0; base < n_items; base += grid, ++round) {
      int w = wg;
      if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
      if (g_mut == 7 && (round & 1) && (grid & 7) == 0) w = (((grid >> 3) - (w >> 3)) << 3) | (w & 7);
      const int bid = base + w;
      Geo g;
      if (bid < n_items) {
        CHECK(bid >= 0 && bid < (int)visited.size(), "work item id %d out of range", bid);
        ++visited[bid];
        if (item_geo(s, n_qtiles, bid, g)) {
          Item it;
          it.id = bid;
          it.len = g.len;
          it.q0 = g.qt * BM;
          it.n_tiles = (g.len + TN - 1) / TN;
          if (s.causal) it.n_tiles = std::min(it.n_tiles, (it.q0 + BM + TN - 1) / TN);
          items.push_back(it);
        }
      }
    }
    if (items.empty()) continue;
    m = Machine();
    m.ipw2 = 2 * ipw;
    // ---- per-wave programs
    std::vector<std::vector<Step>> prog(NW);
    for (int w = 0; w < NW; ++w) {
      auto& P = prog[w];
      const int rblk = w < 4 ? w : 11 - w;
      auto req_tile = [&](int stage, const Item& it, int t) {
        if (t < it.n_tiles) P.push_back({Step::REQ_TILE, stage, it.id, t});
      };
      P.push_back({Step::REQ_Q, items[0].id});
      req_tile(0, items[0], 0);
      req_tile(1, items[0], 1);
      req_tile(2, items[0], 2);
      int in_flight_ok = 0;  // what the wait at the top may leave in flight
      for (size_t k = 0; k < items.size(); ++k) {
        const Item& it = items[k];
        const int q0w = it.q0 + 32 * rblk;
        int H_w = (it.len + 31) / 32;
        if (s.causal) H_w = std::min(H_w, q0w / 32 + 1);
        H_w = std::min(H_w, 2 * it.n_tiles);
        if (q0w >= it.len) H_w = 0;
        const int tail_t = std::max(1, it.n_tiles - (NS - 1));
        P.push_back({Step::WAIT, in_flight_ok});
        P.push_back({Step::USE_Q, it.id});
        P.push_back({Step::BARRIER});
        req_tile(NS - 1, it, NS - 1);
        if (H_w > 0) {
          P.push_back({Step::READ, 0, it.id, 0, "K of half 0"});
          if (1 < H_w) P.push_back({Step::READ, 0, it.id, 0, "K of half 1"});
        }
        for (int t = 0; t < it.n_tiles; ++t) {
          const int TS = t % NS;
          if (t + NS - 1 < it.n_tiles) {
            if (t > 0) {
              P.push_back({Step::WAIT, (g_mut == 1 ? NS - 2 : NS - 3) * 2 * ipw});
              P.push_back({Step::BARRIER});
              req_tile((TS + (g_mut == 3 ? NS - 2 : NS - 1)) % NS, it, t + NS - 1);
            }
          } else if (t == tail_t && g_mut != 4) {
            P.push_back({Step::WAIT, 0});
            P.push_back({Step::BARRIER});
          }
          for (int kb = 0; kb < 2; ++kb) {
            const int h = 2 * t + kb;
            if (h >= H_w) continue;
            // block A: scores of half h + 1 (used when that half exists for this wave)
            if (h + 1 < H_w) {
              const int tk = (h + 1) / 2;
              P.push_back({Step::READ, tk % NS, it.id, tk, "K of the next half"});
            }
            // block B: V of half h; first K fragments of half h + 2
            P.push_back({Step::READ, TS, it.id, t, "V"});
            if (h + 2 < H_w) {
              const int tk = (h + 2) / 2;
              P.push_back({Step::READ, tk % NS, it.id, tk, "first K fragments two halves ahead"});
            }
          }
        }
        P.push_back({Step::BARRIER});
        const bool more = k + 1 < items.size();
        if (more) {
          P.push_back({Step::REQ_Q, items[k + 1].id});
          req_tile(0, items[k + 1], 0);
        }
        // write-out: staging in the last stage, two passes of stores
        const int rows = std::max(0, std::min(32, it.len - q0w));
        // a store instruction covers 64 / CH rows; it is issued when any of its rows exists
        const int per_pass = out_stores_full / 2;
        const int rows_per_store = 32 / per_pass;
        const int live = (rows + rows_per_store - 1) / rows_per_store;
        P.push_back({Step::STAGE_TOUCH, NS - 1});
        P.push_back({Step::STORE, live});
        if (more) req_tile(1, items[k + 1], 1);
        P.push_back({Step::STORE, live});
        if (more) req_tile(2, items[k + 1], 2);
        in_flight_ok = (q0w + 32 <= it.len && more && 2 < items[k + 1].n_tiles) ? out_stores_full / 2 + 2 * ipw : 0;
        if (g_mut == 2 && in_flight_ok) in_flight_ok += 2 * ipw;
        if (g_mut == 8 && more && 2 < items[k + 1].n_tiles) in_flight_ok = out_stores_full / 2 + 2 * ipw;
        // the claim behind that count: exactly the second pass of stores and tile 2 were issued last
        if (in_flight_ok) CHECK(live == per_pass, "full rows but %d of %d store instructions", live, per_pass);
      }
    }
    execute(prog, m, ksteps);
  }
}

// prefill.hip, dense_short_kernel: 4 waves, 128 rows per item, tiles of 32 keys
// in five stages; tile j is requested at the top of position j - 4; at the top
// of position h tiles up to h + 2 must have landed.
namespace short_form {
constexpr int NW = 4, NS = 5, TN = 32, BM = 128;
using Machine = MachineT<NW, NS>;

static void run(const Shape& s, int grid, int ksteps, int ipw, std::vector<int>& visited) {
  const int n_qtiles = (s.max_seqlen + BM - 1) / BM;
  const int n_items = n_qtiles * s.hq * s.batch;
  for (int wg = 0; wg < grid; ++wg) {
    std::vector<Item> items;
    int round = 0;
    for (int base = 0; base < n_items; base += grid, ++round) {
      int w = wg;
      if ((round & 1) && (grid & 7) == 0) w = (((grid >> 3) - 1 - (w >> 3)) << 3) | (w & 7);
      const int bid = base + w;
      Geo g;
      if (bid < n_items) {
        ++visited[bid];
        if (item_geo(s, n_qtiles, bid, g, BM)) {
          Item it;
          it.id = bid;
          it.len = g.len;
          it.q0 = g.qt * BM;
          it.n_tiles = (g.len + TN - 1) / TN;
          if (s.causal) it.n_tiles = std::min(it.n_tiles, (it.q0 + BM + TN - 1) / TN);
          items.push_back(it);
        }
      }
    }
    if (items.empty()) continue;
    Machine m;
    m.ipw2 = 2 * ipw;
    std::vector<std::vector<Step>> prog(NW);
    for (int w = 0; w < NW; ++w) {
      auto& P = prog[w];
      auto req_tile = [&](int stage, const Item& it, int t) {
        if (t < it.n_tiles) P.push_back({Step::REQ_TILE, stage, it.id, t});
      };
      P.push_back({Step::REQ_Q, items[0].id});
      for (int t = 0; t < NS - 1; ++t) req_tile(t, items[0], t);
      for (size_t k = 0; k < items.size(); ++k) {
        const Item& it = items[k];
        const int q0w = it.q0 + 32 * w;
        int H_w = (it.len + 31) / 32;
        if (s.causal) H_w = std::min(H_w, q0w / 32 + 1);
        H_w = std::min(H_w, it.n_tiles);
        if (q0w >= it.len) H_w = 0;
        const int tail_h = std::max(1, it.n_tiles - (NS - 1));
        // item top: tile 3, when it exists, is the youngest request and may stay in flight
        int allow = (NS - 2 < it.n_tiles) ? 2 * ipw : 0;
        if (g_mut == 11) allow = 2 * ipw;
        P.push_back({Step::WAIT, allow});
        P.push_back({Step::USE_Q, it.id});
        P.push_back({Step::BARRIER});
        req_tile(NS - 1, it, NS - 1);
        if (H_w > 0) P.push_back({Step::READ, 0, it.id, 0, "K of tile 0"});
        for (int h = 0; h < it.n_tiles; ++h) {
          if (h > 0) {
            if (h + NS - 1 < it.n_tiles) {
              P.push_back({Step::WAIT, (g_mut == 12 ? NS - 3 : NS - 4) * 2 * ipw});
              P.push_back({Step::BARRIER});
              req_tile((h + NS - 1) % NS, it, h + NS - 1);
            } else if (h == tail_h) {
              P.push_back({Step::WAIT, 0});
              P.push_back({Step::BARRIER});
            }
          }
          if (h >= H_w) continue;
          if (h + 1 < H_w) P.push_back({Step::READ, (h + 1) % NS, it.id, h + 1, "K of the next tile"});
          P.push_back({Step::READ, h % NS, it.id, h, "V"});
          if (h + 2 < H_w) P.push_back({Step::READ, (h + 2) % NS, it.id, h + 2, "first K fragments two tiles ahead"});
        }
        P.push_back({Step::BARRIER});
        const bool more = k + 1 < items.size();
        if (more) {
          P.push_back({Step::REQ_Q, items[k + 1].id});
          req_tile(0, items[k + 1], 0);
        }
        const int rows = std::max(0, std::min(32, it.len - q0w));
        P.push_back({Step::STAGE_TOUCH, NS - 1});
        P.push_back({Step::STORE, rows > 0 ? 2 : 0});
        if (more) req_tile(1, items[k + 1], 1);
        P.push_back({Step::STORE, rows > 0 ? 2 : 0});
        if (more) {
          req_tile(2, items[k + 1], 2);
          req_tile(3, items[k + 1], 3);
        }
      }
    }
    execute(prog, m, ksteps);
  }
}
}  // namespace short_form

static void test(std::mt19937& rng) {
  int cases = 0;
  for (int rep = 0; rep < 200; ++rep) {
    Shape s;
    s.causal = rng() % 4 != 0;
    s.hkv = 1 + rng() % 4;
    s.hq = s.hkv * (1 + rng() % 3);
    s.batch = (rep % 3 == 0) ? 8 / std::min(8, s.hkv) * (1 + rng() % 2) : 1 + rng() % 5;   // some shapes with units % 8 == 0
    const int maxlen = 1 + rng() % 1400;
    for (int b = 0; b < s.batch; ++b) s.lens.push_back(rng() % 5 == 0 ? (int)(rng() % 3) : 1 + (int)(rng() % maxlen));
    s.max_seqlen = rep % 7 == 0 ? std::max(1, maxlen / 2) : maxlen;   // a bound below the longest sequence cuts it
    const int n_qtiles = (s.max_seqlen + BM - 1) / BM;
    const int n_items = n_qtiles * s.hq * s.batch;
    for (int grid : {1, 3, 8, 16, 256}) {
      if (grid > n_items) grid = n_items;
      for (int d : {64, 96, 128}) {
        // K fragments of a row, tile loads per wave and tensor (rows of 96 are padded to 128), output stores of 32 full rows
        const int ksteps = d / 16, ipw = d == 64 ? 1 : 2, out_stores = d == 64 ? 4 : 8;
        Machine m;
        std::vector<int> visited(n_items, 0);
        run(s, grid, ksteps, ipw, out_stores, m, visited);
        for (int i = 0; i < n_items; ++i) CHECK(visited[i] == 1, "work item %d of %d visited %d times (grid %d)", i, n_items, visited[i], grid);
        ++cases;
      }
    }
    // the short form of the same kernel: 128-row items, two or three workgroups per CU
    {
      const int nq = (s.max_seqlen + short_form::BM - 1) / short_form::BM;
      const int ni = nq * s.hq * s.batch;
      for (int grid : {1, 5, 16, 768}) {
        if (grid > ni) grid = ni;
        for (int d : {64, 128}) {   // (128: two tile loads per wave and tensor instead of one; the kernel is generic)
          std::vector<int> visited(ni, 0);
          short_form::run(s, grid, d / 16, d == 64 ? 1 : 2, visited);
          for (int i = 0; i < ni; ++i) CHECK(visited[i] == 1, "short form: work item %d of %d visited %d times (grid %d)", i, ni, visited[i], grid);
          ++cases;
        }
      }
    }
    // the item map is a bijection onto (sequence, q head, q tile)
    std::set<long long> seen;
    for (int bid = 0; bid < n_items; ++bid) {
      Geo g;
      item_geo(s, n_qtiles, bid, g);
      CHECK(g.b >= 0 && g.b < s.batch && g.h >= 0 && g.h < s.hq && g.qt >= 0 && g.qt < n_qtiles && g.kvh == g.h / (s.hq / s.hkv),
            "item %d maps outside the problem", bid);
      seen.insert(((long long)g.b * s.hq + g.h) * n_qtiles + g.qt);
    }
    CHECK((int)seen.size() == n_items, "item map is not one-to-one: %zu of %d", seen.size(), n_items);
  }
  std::printf("dense walk: %d runs\n", cases);
}
}  // namespace dense

// ------------------------------------------------------------------ block-sparse
namespace sparse {
// prefill.hip, sparse_kernel: two wavefronts walk the tiles of a CSR row (a
// listed 64-key block is two 32-key tiles).  K tiles run one position ahead of
// V tiles and each tensor has a ring of two stages; the block list is held 64
// entries at a time in two registers and read with a lane index.
constexpr int NW = 2;
struct Stage {
  int tile = -1, block = -1, issued_in = -1;
  bool landed[NW] = {}, published = false;
};
struct Machine {
  Stage k[2], v[2];
  int interval = 0;
  std::vector<const Stage*> read_now;
  std::vector<std::pair<Stage*, int>> in_flight[NW];  // (stage, tile) per wave, in issue order
  void request(int w, Stage& s, int tile, int block) {
    if (s.tile != tile || s.issued_in != interval) {
      s.tile = tile; s.block = block; s.issued_in = interval; s.published = false;
      for (bool& l : s.landed) l = false;
    }
    for (const Stage* r : read_now) CHECK(r != &s, "tile %d is requested into a stage that is read in the same barrier interval", tile);
    in_flight[w].push_back({&s, tile});
  }
  void wait_all(int w) {
    for (auto& f : in_flight[w])
      if (f.first->tile == f.second) f.first->landed[w] = true;
    in_flight[w].clear();
  }
  void read(int w, const Stage& s, int tile, int block, const char* what) {
    CHECK(s.tile == tile && s.block == block, "wave %d reads %s of tile %d (block %d), the stage holds tile %d (block %d)", w, what, tile, block, s.tile, s.block);
    CHECK(s.published && s.issued_in < interval, "wave %d reads %s of tile %d before it is published", w, what, tile);
    read_now.push_back(&s);
  }
  void barrier() {
    ++interval;
    read_now.clear();
    for (Stage* s : {&k[0], &k[1], &v[0], &v[1]})
      if (s->tile >= 0 && s->landed[0] && s->landed[1]) s->published = true;
  }
};

static void walk(const std::vector<int>& cols) {
  const int n_blk = (int)cols.size(), n_tiles = 2 * n_blk;
  if (n_tiles == 0) return;
  Machine m;
  // the list registers of a wave: entry 64 * chunk + lane, the chunk walked and the one behind it
  auto load_cols = [&](int chunk) {
    std::vector<int> r(64, 0);
    for (int l = 0; l < 64; ++l)
      if (chunk * 64 + l < n_blk) r[l] = cols[chunk * 64 + l];
    return r;
  };
  struct WaveRegs {
    int col_chunk = 0;
    std::vector<int> col_cur, col_nxt;
    int blkC = 0, blkN = 0;
    bool hasN = false;
  } wr[NW];
  for (auto& r : wr) { r.col_cur = load_cols(0); r.col_nxt = load_cols(1); }
  // prologue: K and V of tile 0, K of tile 1; full wait; barrier; scores of tile 0; barrier
  for (int w = 0; w < NW; ++w) {
    wr[w].blkC = wr[w].col_cur[0];
    m.request(w, m.k[0], 0, wr[w].blkC);
    m.request(w, m.v[0], 0, wr[w].blkC);
    m.request(w, m.k[1], 1, wr[w].blkC);
    m.wait_all(w);
  }
  m.barrier();
  for (int w = 0; w < NW; ++w) m.read(w, m.k[0], 0, cols[0], "K");
  if (g_mut != 9) m.barrier();
  for (int h = 0; h < n_tiles; ++h) {
    const int J = h & 1;
    const bool last = h == n_tiles - 1;
    for (int w = 0; w < NW; ++w) {
      WaveRegs& r = wr[w];
      if (J == 0) {
        const int bn = (h >> 1) + 1;
        r.hasN = bn < n_blk;
        if (r.hasN) {
          if ((bn >> 6) != r.col_chunk) {
            ++r.col_chunk;
            r.col_cur = r.col_nxt;
            r.col_nxt = load_cols(r.col_chunk + (g_mut == 10 ? 0 : 1));
          }
          r.blkN = r.col_cur[bn & 63];
        }
      }
      const bool has1 = J == 0 ? true : r.hasN, has2 = r.hasN;
      if (!last) {
        // K of tile h + 2 into the K stage of tile h, V of tile h + 1 into the V stage of tile h - 1
        if (has2) m.request(w, m.k[J], h + 2, r.blkN);
        if (has1) m.request(w, m.v[J ^ 1], h + 1, J == 0 ? r.blkC : r.blkN);
        m.read(w, m.k[J ^ 1], h + 1, cols[(h + 1) >> 1], "K");
      }
      m.read(w, m.v[J], h, cols[h >> 1], "V");
      if (!last) {
        if (J == 1) r.blkC = r.blkN;
        m.wait_all(w);
      }
    }
    if (!last) m.barrier();
  }
}

static void test(std::mt19937& rng) {
  int cases = 0;
  for (int n = 0; n <= 400; ++n) {
    std::vector<int> cols(n);
    for (auto& c : cols) c = (int)(rng() % 100000);   // any block ids: the walk must name them in list order
    walk(cols);
    ++cases;
  }
  std::printf("block-sparse walk: %d lists\n", cases);
}
}  // namespace sparse

// ------------------------------------------------------------------ softmax
namespace softmax {
// prefill.hip: probabilities of a half (16 scores per lane of a row here: the
// whole row is one "lane") are taken against the reference point the row
// already has; the reference moves to the exact running maximum only when a
// half's partial sum passes 4096 or is not finite.  o and lse must not depend
// on it.
static void test(std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  int fixes = 0, cases = 0;
  for (int rep = 0; rep < 300; ++rep) {
    const int halves = 1 + rng() % 12, D = 4;
    const float scale = 0.125f * 1.44269504f;
    const float growth = rep % 3 == 0 ? 40.f : (rep % 3 == 1 ? 4.f : 0.f);   // scores that keep growing along the keys
    std::vector<float> sc(halves * 32), v(halves * 32 * D);
    for (int i = 0; i < halves * 32; ++i) sc[i] = nd(rng) * 8.f + growth * (float)(i / 32);
    for (auto& x : v) x = nd(rng);
    // reference: plain softmax in double
    double mx = -1e300;
    for (float x : sc) mx = std::max(mx, (double)x * scale);
    double den = 0;
    std::vector<double> o_ref(D, 0.0);
    for (int i = 0; i < halves * 32; ++i) {
      const double p = std::exp2((double)sc[i] * scale - mx);
      den += p;
      for (int d = 0; d < D; ++d) o_ref[d] += p * v[i * D + d];
    }
    const double lse_ref = mx + std::log2(den);
    // running reference point
    float m = -INFINITY, m_neg = 0.f, l = 0.f;
    std::vector<float> o(D, 0.f);
    for (int h = 0; h < halves; ++h) {
      float p[32], rs = 0.f;
      auto exact_fix = [&]() {
        float hm = sc[h * 32];
        for (int i = 1; i < 32; ++i) hm = std::max(hm, sc[h * 32 + i]);
        const float m_new = std::max(m, hm * scale);
        const float alpha = std::exp2(m - m_new);
        l *= alpha;
        for (auto& x : o) x *= alpha;
        m = m_new;
        m_neg = -m_new;
        rs = 0.f;
        for (int i = 0; i < 32; ++i) { p[i] = std::exp2(std::fma(sc[h * 32 + i], scale, m_neg)); rs += p[i]; }
        ++fixes;
      };
      if (h == 0) {
        exact_fix();
      } else {
        for (int i = 0; i < 32; ++i) { p[i] = std::exp2(std::fma(sc[h * 32 + i], scale, m_neg)); rs += p[i]; }
        if (!(rs <= 4096.f) && g_mut != 6) exact_fix();
      }
      l += rs;
      for (int i = 0; i < 32; ++i)
        for (int d = 0; d < D; ++d) o[d] += p[i] * v[(h * 32 + i) * D + d];
    }
    const float lse = m + std::log2(l);
    CHECK(std::isfinite(lse) && std::fabs(lse - lse_ref) <= 1e-3 * std::max(1.0, std::fabs(lse_ref)), "lse %g against %g", lse, lse_ref);
    for (int d = 0; d < D; ++d) {
      const double got = o[d] / l, want = o_ref[d] / den;
      CHECK(std::fabs(got - want) <= 2e-4 * std::max(1.0, std::fabs(want)), "o[%d] %g against %g", d, got, want);
    }
    ++cases;
  }
  CHECK(fixes > 300, "the growing scores never moved the reference point");
  std::printf("softmax reference point: %d rows, %d moves of the reference\n", cases, fixes);
}
}  // namespace softmax

// ------------------------------------------------------------------ decode
namespace decode {
struct WindowList {
  int n_sink, tail0, cnt;
  int block(int e) const { return e < n_sink ? e : tail0 + (e - n_sink); }
};
// decode.hip: window_list
static WindowList window_list(int len, int wg, int wl) {
  const int nblk = (len + 63) / 64;
  WindowList w;
  w.n_sink = std::min((wg + 63) / 64, nblk);
  w.tail0 = std::max(std::max(len - wl, 0) / 64, g_mut == 5 ? 0 : w.n_sink);
  w.cnt = w.n_sink + std::max(nblk - w.tail0, 0);
  return w;
}

static void test(std::mt19937& rng) {
  int cases = 0;
  for (int rep = 0; rep < 20000; ++rep) {
    const int len = rep < 700 ? rep : 1 + (int)(rng() % 20000);
    const int wg = (rep % 5 == 0) ? (int)(rng() % 700) : 64 * (1 + (int)(rng() % 4));
    const int wl = (int)(rng() % 3) == 0 ? (int)(rng() % 200) : (int)(rng() % 9000);
    const WindowList w = window_list(len, wg, wl);
    // blocks that hold at least one attended token: k < wg or k >= len - wl, k < len
    std::set<int> want;
    for (int k = 0; k < len; ++k)
      if (k < wg || k >= len - wl) want.insert(k / 64);
    std::set<int> got;
    int prev = -1;
    for (int e = 0; e < w.cnt; ++e) {
      const int blk = w.block(e);
      CHECK(blk > prev, "window list not ascending / unique at entry %d (len %d, wg %d, wl %d)", e, len, wg, wl);
      CHECK(blk >= 0 && blk < (len + 63) / 64, "window list names block %d of a sequence of %d tokens", blk, len);
      prev = blk;
      got.insert(blk);
    }
    // the list may hold blocks whose tokens are all masked by the window (the block of token len - wl when
    // wl = 0, say); it must hold every block with an attended token
    for (int b : want) CHECK(got.count(b), "block %d missing (len %d, wg %d, wl %d)", b, len, wg, wl);
    CHECK((int)got.size() <= (int)want.size() + 1, "window list holds %zu blocks for %zu attended ones", got.size(), want.size());
    const int cap = (wg + 63) / 64 + (wl + 63) / 64 + 1;  // what the host sizes max_blocks with
    CHECK(w.cnt <= cap, "window list of %d entries exceeds its bound %d (len %d, wg %d, wl %d)", w.cnt, cap, len, wg, wl);
    ++cases;
  }
  // dense form: the live chunks of a ragged batch, numbered consecutively and dealt round-robin
  for (int rep = 0; rep < 300; ++rep) {
    const int batch = 1 + rng() % 70, hkv = 1 + rng() % 4, gslices = 1 + rng() % 3, split = 64 * (1 + rng() % 32);
    std::vector<int> lens(batch);
    int maxlen = 1;
    for (auto& l : lens) { l = rng() % 6 == 0 ? 0 : (int)(rng() % 40000); maxlen = std::max(maxlen, l); }
    const int n_splits = (maxlen + split - 1) / split;
    auto chunks_of = [&](int b) { return b >= batch ? 0 : std::max(0, std::min((lens[b] + split - 1) / split, n_splits)); };
    long long total = 0;
    for (int b = 0; b < batch; ++b) total += chunks_of(b);
    const long long items = total * hkv * gslices;
    const int grid = 1 + rng() % 2048;
    std::set<long long> seen;
    for (int wgp = 0; wgp < grid; ++wgp)
      for (long long g = wgp; g < items; g += grid) {
        const int kv_slices = hkv * gslices;
        const int t = (int)(g / kv_slices), kvs = (int)(g % kv_slices);
        int b = 0, first = 0, seen_chunks = 0;
        for (; b < batch; ++b) {
          const int c = chunks_of(b);
          if (t < seen_chunks + c) { first = seen_chunks; break; }
          seen_chunks += c;
        }
        CHECK(b < batch, "chunk %d belongs to no sequence", t);
        const int chunk = t - first;
        CHECK(chunk * split < lens[b], "chunk %d of sequence %d starts past its end", chunk, b);
        seen.insert(((long long)b * n_splits + chunk) * kv_slices + kvs);
      }
    CHECK((long long)seen.size() == items, "%zu of %lld (chunk, kv-head, slice) items dealt", seen.size(), items);
    ++cases;
  }
  std::printf("decode lists and chunks: %d cases\n", cases);
}
}  // namespace decode

// ------------------------------------------------------- window walk (prefill)
// dense_short_kernel<T, D, WIN = true>: a 128-row item of the two-window form
// walks the tiles (32 keys) of the first win_global keys, then the band that
// ends at its diagonal block.  Restated here: the item's walk (next_item), the
// key of a position (key_of), the positions a wave works on (H_w) and the mask
// of a tile (mask_half).  Checked against the rule itself - key k is visible to
// query r iff k <= r and (r - k < wl or k < wg) - for every row of every wave.
namespace window_walk {
constexpr int TN = 32, BM = 128, NW = 4;
struct Walk {
  int n_sink, skip, n_tiles;
  int key_of(int j) const { return (j + (j >= n_sink ? skip : 0)) * TN; }
};
static Walk item_walk(int q0, int len, int wl, int wg) {
  Walk w;
  w.n_tiles = std::min((len + TN - 1) / TN, (q0 + BM + TN - 1) / TN);  // causal
  const int t0 = std::max(q0 - wl + 1, 0) / TN;
  w.n_sink = g_mut == 14 ? (wg + TN - 1) / TN : std::min((wg + TN - 1) / TN, t0);
  w.skip = t0 - w.n_sink;
  w.n_tiles -= w.skip;
  return w;
}
static int wave_positions(const Walk& w, int q0w, int len) {
  int h = std::min((len + 31) / 32, q0w / 32 + 1);
  if (g_mut != 13) h -= w.skip;
  h = std::min(h, w.n_tiles);
  return q0w >= len ? 0 : h;
}
// is key k0h + off masked for the lane whose query is `row` (already cut at len - 1)?
static bool masked(int k0h, int off, int row, int q0w, int len, int wl, int wg, bool& edge) {
  edge = (k0h + 32 > len) || (k0h + 31 > q0w);
  if (g_mut != 15) edge = edge || (k0h <= q0w + 31 - wl && k0h + 31 >= wg);
  if (!edge) return false;
  const int t = row - k0h;
  const int below = t - wl, sink = wg - k0h;
  return off > t || (off <= below && off >= sink);
}

static void test(std::mt19937& rng) {
  int cases = 0;
  for (int rep = 0; rep < 6000; ++rep) {
    const int len = rep < 300 ? 1 + rep : 1 + (int)(rng() % 5000);
    const int wl = rep % 7 == 0 ? 1 + (int)(rng() % 40) : 1 + (int)(rng() % 3000);
    const int wg = rep % 3 == 0 ? 0 : (int)(rng() % 400);
    const int n_items = (len + BM - 1) / BM;
    const int item = (int)(rng() % n_items), q0 = item * BM;
    const Walk w = item_walk(q0, len, wl, wg);
    CHECK(w.n_tiles >= 1, "item at row %d walks %d tiles (len %d, wl %d, wg %d)", q0, w.n_tiles, len, wl, wg);
    int prev = -1;
    for (int j = 0; j < w.n_tiles; ++j) {
      const int k0 = w.key_of(j);
      CHECK(k0 > prev && k0 < len, "position %d is tile %d after tile %d (len %d, q0 %d, wl %d, wg %d)", j, k0 / TN, prev / TN, len, q0, wl, wg);
      prev = k0;
    }
    for (int wave = 0; wave < NW; ++wave) {
      const int q0w = q0 + 32 * wave;
      const int H = wave_positions(w, q0w, len);
      CHECK(H >= 0 && H <= w.n_tiles, "wave %d works on %d of %d positions", wave, H, w.n_tiles);
      if (q0w >= len) continue;
      // no position that lies wholly above the wave's diagonal is worked on
      CHECK(H >= 1 && w.key_of(H - 1) <= std::min(q0w + 31, len - 1), "wave %d works on %d positions, the last one from key %d on, above its rows %d.. (skip %d)",
            wave, H, H >= 1 ? w.key_of(H - 1) : -1, q0w, w.skip);
      for (int lq = 0; lq < 32; ++lq) {
        const int row = std::min(q0w + lq, len - 1);   // rows past the end repeat the last one
        // what the walk lets this row see
        std::vector<char> seen(len, 0);
        for (int j = 0; j < H; ++j) {
          const int k0h = w.key_of(j);
          for (int off = 0; off < 32; ++off) {
            bool edge;
            const bool m = masked(k0h, off, row, q0w, len, wl, wg, edge);
            if (!m) {
              CHECK(k0h + off < len, "row %d sees key %d of a sequence of %d tokens", row, k0h + off, len);
              if (k0h + off < len) seen[k0h + off] = 1;
            }
          }
        }
        for (int k = 0; k < len; ++k) {
          const bool want = k <= row && (row - k < wl || k < wg);
          CHECK((bool)seen[k] == want, "row %d %s key %d (len %d, q0 %d, wave %d, wl %d, wg %d, sink %d skip %d tiles %d H %d)",
                row, want ? "misses" : "wrongly sees", k, len, q0, wave, wl, wg, w.n_sink, w.skip, w.n_tiles, H);
          if ((bool)seen[k] != want) break;
        }
      }
    }
    ++cases;
  }
  std::printf("window walk: %d items\n", cases);
}
}  // namespace window_walk

int main(int argc, char** argv) {
  if (argc > 1) g_mut = std::atoi(argv[1]);
  std::mt19937 rng(12345);
  if (g_mut != 5 && g_mut != 6) dense::test(rng);   // (those two mistakes sit in the other parts)
  sparse::test(rng);
  softmax::test(rng);
  decode::test(rng);
  window_walk::test(rng);
  if (g_fail) {
    std::printf("%d check(s) failed\n", g_fail);
    return 1;
  }
  std::printf("host model ok\n");
  return 0;
}
