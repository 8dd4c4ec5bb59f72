// Host-only robustness driver for the plan builder (built by tests/test_host_sanitizers.py with
// -fsanitize=address,undefined): reads flat int32 tables from a file, builds the plan, dry-runs it,
// decides a geometry, then repeats with randomly corrupted copies of the tables.  Any invalid table
// must come back as an error code -- never as a crash, an out-of-bounds access or undefined behaviour.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "plan.h"

namespace mscclx { void destroy_device_state(DeviceState*) {} }  // no device half in this build

static int run_once(int nranks, const std::vector<int32_t>& rc, const std::vector<int32_t>& tbs, const std::vector<int32_t>& ops, bool expect_ok, int variants) {
  mscclx_plan_desc d{nranks, (int32_t)(tbs.size() / MSCCLX_TB_COLS), (int32_t)(ops.size() / MSCCLX_OP_COLS), rc.data(), tbs.data(), ops.data()};
  mscclx_plan* p = nullptr;
  int rc_create = mscclx_plan_create(&d, &p);
  if (rc_create != MSCCLX_OK) {
    if (expect_ok) { fprintf(stderr, "valid tables rejected: %s\n", mscclx_last_error()); return 1; }
    return 0;
  }
  (void)mscclx_plan_simulate(p, 0);
  (void)mscclx_plan_simulate(p, 2);
  (void)mscclx_plan_algorithmic_units(p);
  const int capacity[mscclx::kThreadChoices] = {4096, 2048, 1024, 512, 256};
  mscclx::Geometry g;
  for (int variant = 0; variant < variants; ++variant)  // 0 automatic, 1 LL lines, 2 explicit knobs with staging
  for (size_t chunk : {(size_t)4, (size_t)4096, (size_t)(1 << 20) + 16, (size_t)3 << 20}) {
    mscclx_config cfg = {};
    if (variant == 1) cfg.protocol = MSCCLX_PROTO_LL;
    if (variant == 2) { cfg.staging = 1; cfg.slices = 3; cfg.piece_bytes = 4096; }
    int r = mscclx::decide_geometry(*p, chunk, MSCCLX_F32, cfg, 256, capacity, 1ull << 30, &g);
    if (r == MSCCLX_OK) {
      size_t hosted = g.ctx_tb.size();
      if (hosted != p->tbs.size() * (size_t)g.slices || g.wg_begin.back() != (int32_t)hosted) { fprintf(stderr, "hosting table does not cover every context\n"); return 1; }
    } else if (expect_ok && r != MSCCLX_ERR_DEADLOCK && r != MSCCLX_ERR_CAPACITY && r != MSCCLX_ERR_UNSUPPORTED && r != MSCCLX_ERR_INVALID_ARG) {
      fprintf(stderr, "geometry failed on valid tables: %s\n", mscclx_last_error());
      return 1;
    }
  }
  mscclx_plan_destroy(p);
  return 0;
}

int main(int argc, char** argv) {
  if (argc < 3) { fprintf(stderr, "usage: %s tables.bin mutations\n", argv[0]); return 2; }
  FILE* f = fopen(argv[1], "rb");
  if (!f) return 2;
  int32_t hdr[3];
  if (fread(hdr, 4, 3, f) != 3) return 2;
  std::vector<int32_t> rc((size_t)hdr[0] * 3), tbs((size_t)hdr[1] * MSCCLX_TB_COLS), ops((size_t)hdr[2] * MSCCLX_OP_COLS);
  if (fread(rc.data(), 4, rc.size(), f) != rc.size() || fread(tbs.data(), 4, tbs.size(), f) != tbs.size() ||
      fread(ops.data(), 4, ops.size(), f) != ops.size()) return 2;
  fclose(f);
  if (run_once(hdr[0], rc, tbs, ops, true, 3)) return 1;
  std::mt19937 rng(12345);
  const int mutations = atoi(argv[2]);
  const int32_t nasty[] = {-2147483647 - 1, -2, -1, 0, 1, 2, 7, 63, 64, 65, 1000, 2147483647};
  for (int m = 0; m < mutations; ++m) {
    auto a = rc, b = tbs, c = ops;
    const int edits = 1 + rng() % 3;
    for (int e = 0; e < edits; ++e) {
      std::vector<int32_t>& v = (rng() % 8 == 0) ? a : (rng() % 3 == 0 ? b : c);
      if (v.empty()) continue;
      v[rng() % v.size()] = (rng() % 2) ? nasty[rng() % 12] : (int32_t)(rng() % 40) - 4;
    }
    if (run_once(hdr[0], a, b, c, false, m % 8 == 0 ? 3 : 1)) return 1;
  }
  printf("ok: %d mutated tables handled\n", mutations);
  return 0;
}
