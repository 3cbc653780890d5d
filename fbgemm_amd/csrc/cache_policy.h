// Which entry a bounded cache gives up: the least recently used one among those that may go.
// Entries a captured HIP graph may hold (a forward under stream capture has touched them) may
// not: the graph replays raw device addresses. With every entry held, nothing goes and the
// cache grows past its bound. Host code only; shared by the work-list cache of a plan
// (c_api.cpp) and the operator's cache of plans (torch_op.cpp).
#pragma once

namespace fbgemm_amd {

// `held(entry)`: the entry must stay; `last_use(entry)`: a counter that grows with every use.
// Returns m.end() when every entry must stay.
template <typename Map, typename Held, typename LastUse>
typename Map::iterator least_recently_used_not_held(Map& m, Held held, LastUse last_use) {
  auto victim = m.end();
  for (auto it = m.begin(); it != m.end(); ++it)
    if (!held(it->second) && (victim == m.end() || last_use(it->second) < last_use(victim->second))) victim = it;
  return victim;
}

} // namespace fbgemm_amd
