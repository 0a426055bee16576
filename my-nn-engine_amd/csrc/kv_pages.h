// Page table of a set of sequences over a pool of KV pages (kv_pages.hip): what the executor needs of it.
#pragma once
#include "kernels.h"

namespace mynn {

// pages for rows [0, rows) of every sequence of the set, taken from the pool as needed and published to the device
// table (synchronous); MYNN_ERR_TOO_LONG beyond the set's rows, MYNN_ERR_NO_PAGES when the pool runs dry
int kv_pages_reserve(mynn_kv_pages *ps, long rows);
KvPaging kv_pages_paging(const mynn_kv_pages *ps);
int kv_pages_batch(const mynn_kv_pages *ps);
int kv_pages_pool_pages(const mynn_kv_pages *ps);

}  // namespace mynn
