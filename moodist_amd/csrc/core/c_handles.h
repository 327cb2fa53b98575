// The structs behind the opaque handles of include/moodist_core.h, shared by the files that
// hand them out (c_api.cc, plugin.cc).
#pragma once

#include <memory>

#include "moodist_core.h"
#include "processgroup.h"

struct moodist_world {
  std::shared_ptr<moodist::World> impl;
};
struct moodist_work {
  std::shared_ptr<moodist::Collective> c;
};
struct moodist_op {
  moodist::ProcessGroup* pg;
  std::shared_ptr<moodist::CompiledOp> op;
};
struct moodist_future {
  std::shared_ptr<moodist::Collective> c;
};
