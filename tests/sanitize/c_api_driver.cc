// Walks the C ABI of the host core through handle lifetimes that a binding can produce:
// collectives left incomplete, works and ops destroyed before and after their world, plan
// accessors with out-of-range indices, launches that fail for want of a device or of the
// kernel library.  Built with -fsanitize=address,undefined by tests/test_sanitize_cpu.py.
#include "moodist_core.h"
#include <cstdio>
#include <cstring>
#include <vector>
static moodist_tensor fake(int64_t numel, int dtype = 6, int itemsize = 4) {
  moodist_tensor t{}; t.data = (void*)0x10000; t.numel = numel; t.itemsize = itemsize; t.dtype = dtype; t.device = 0; t.contiguous = 1; t.ndim = 1; t.shape[0] = numel; return t;
}
int main() {
  std::printf("version ok %d\n", moodist_core_check_version(MOODIST_CORE_API_VERSION));
  for (int round = 0; round < 3; ++round) {
    moodist_world* w = nullptr;
    if (moodist_world_create(4, 0, &w)) { std::printf("create: %s\n", moodist_last_error()); return 1; }
    std::vector<moodist_work*> works;
    for (int r = 0; r < (round == 0 ? 3 : 4); ++r) {
      moodist_pg* pg = moodist_world_group(w, r);
      moodist_tensor in = fake(16), out = fake(4);
      moodist_work* wk = nullptr;
      int rc = moodist_pg_reduce_scatter(pg, &out, &in, 0, nullptr, 0.0f, &wk);
      if (rc) std::printf("round %d rank %d: %s\n", round, r, moodist_last_error());
      if (wk) works.push_back(wk);
    }
    for (auto* wk : works) { int rc = moodist_work_wait(wk); if (rc) std::printf("wait: %s\n", moodist_last_error()); std::printf("completed %d\n", moodist_work_is_completed(wk)); }
    // a list of all_gathers as one collective: left incomplete in round 0, launched (and failing
    // for want of a device) otherwise; a rank that brings another list; things kept alive for it
    {
      std::vector<moodist_work*> many;
      static int released = 0;
      for (int r = 0; r < (round == 0 ? 2 : 4); ++r) {
        moodist_pg* pg = moodist_world_group(w, r);
        moodist_tensor ins[3] = {fake(4), fake(6), fake(r == 3 && round == 2 ? 9 : 10)};
        moodist_tensor outs[3] = {fake(16), fake(24), fake(r == 3 && round == 2 ? 36 : 40)};
        moodist_work* wk = nullptr;
        int rc = moodist_pg_all_gather_many(pg, r % 2 ? outs : nullptr, ins, 3, nullptr, &wk);
        if (rc) std::printf("round %d rank %d many: %s\n", round, r, moodist_last_error());
        if (wk) many.push_back(wk);
        moodist_pg_keep_alive(pg, new int(r), [](void* p) { delete (int*)p; ++released; });
      }
      for (int r = 0; r < (round == 0 ? 1 : 4); ++r) {
        moodist_tensor ts[2] = {fake(16), fake(r == 2 && round == 1 ? 25 : 24)};
        moodist_work* wk = nullptr;
        int rc = moodist_pg_allreduce_many(moodist_world_group(w, r), ts, 2, 0, nullptr, 0.0f, &wk);
        if (rc) std::printf("round %d rank %d allreduce list: %s\n", round, r, moodist_last_error());
        if (wk) many.push_back(wk);
      }
      for (auto* wk : many) { moodist_work_wait(wk); moodist_work_destroy(wk); }
      std::printf("round %d: %d kept objects released so far\n", round, released);
    }
    // compile + plan accessors
    int shape[1] = {8};
    int in_ranks[1] = {0}, in_off[1] = {0}, in_shape[1] = {8};
    int out_ranks[4] = {0, 1, 2, 3}, out_off[4] = {0, 2, 4, 6}, out_shape[4] = {2, 2, 2, 2};
    std::vector<moodist_op*> ops;
    for (int r = 0; r < 4; ++r) {
      moodist_op* op = nullptr;
      int rc = moodist_compile_op_full(moodist_world_group(w, r), shape, 1, 6, in_ranks, in_off, in_shape, 1, out_ranks, out_off, out_shape, 4, &op);
      if (rc) std::printf("compile: %s\n", moodist_last_error());
      if (op) ops.push_back(op);
    }
    for (auto* op : ops) {
      int64_t n = moodist_op_plan_count(op, 0);
      for (int64_t i = 0; i < n; ++i) { int64_t r[6]; moodist_op_plan_read(op, (size_t)i, r); }
      char buf[256];
      for (int rcv = -1; rcv < 6; ++rcv) moodist_op_plan_message(op, rcv, buf, sizeof(buf));
      int64_t tmp[3]; moodist_op_plan_copy(op, 1, 99, tmp, 3); moodist_op_plan_size(op, 3, 99);
    }
    if (round == 1) { for (auto* wk : works) moodist_work_destroy(wk); works.clear(); }
    if (round == 2) { for (auto* op : ops) moodist_op_destroy(op); ops.clear(); }
    moodist_world_destroy(w);   // with handles still alive in some rounds
    for (auto* wk : works) moodist_work_destroy(wk);
    for (auto* op : ops) moodist_op_destroy(op);
  }
  std::puts("c api driver done");
  return 0;
}
