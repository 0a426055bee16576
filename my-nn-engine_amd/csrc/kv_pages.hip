// Paged KV cache: a pool of fixed-size pages shared by any number of sequence sets, and the page table of one set.
//
// The reference keeps one contiguous [batch, Hkv, max_seq, D] buffer per layer and cache side
// (crates/llm/src/session.rs:284-394), reserved in full when the session is made.  Here the buffers of a layer can
// instead be pools [n_pages, Hkv, P, D] (P rows per page, a power of two): a page holds P consecutive rows of every kv
// head of ONE sequence in every layer, the same page number in each layer's K and V pool.  Sessions of different and
// growing lengths then share the memory, and a session takes a page only when its sequences reach it.
//
// Host side only: the pool is a free list of page numbers (the device buffers belong to the caller, like every other
// session-state buffer of the boundary), a page set is the table [batch, pages_per_seq] of one executor pair (prefill +
// decode), mirrored in device memory where the kernels read it.  A page the table does not map holds -1; the kernels
// never look at entries beyond the rows an executor has reserved, and the executor reserves before it launches.
#include <cstring>
#include <mutex>
#include <vector>

#include "kv_pages.h"

using namespace mynn;

struct mynn_kv_pool {
    std::mutex mu;
    std::vector<int32_t> free_list;  // taken from the back; starts as n_pages-1 .. 0 so that pages go out in rising order
    int n_pages = 0, page_rows = 0;
    int sets = 0;  // page sets alive on this pool
};

struct mynn_kv_pages {
    mynn_kv_pool *pool = nullptr;
    int batch = 0, pages_per_seq = 0, shift = 0;
    int mapped = 0;                // pages mapped per sequence (all sequences of a set grow together)
    std::vector<int32_t> host;     // [batch, pages_per_seq], -1 = not mapped
    int32_t *dev = nullptr;
};

namespace mynn {

int kv_pages_reserve(mynn_kv_pages *ps, long rows) {
    MYNN_REQUIRE(ps, MYNN_ERR_INVALID, "kv_pages_reserve: null page set");
    const int P = 1 << ps->shift;
    MYNN_REQUIRE(rows >= 0 && rows <= (long)ps->pages_per_seq * P, MYNN_ERR_TOO_LONG,
                 "kv_pages_reserve: %ld rows exceed %d pages of %d rows", rows, ps->pages_per_seq, P);
    const int need = (int)((rows + P - 1) >> ps->shift);
    if (need <= ps->mapped) return 0;
    const int take = (need - ps->mapped) * ps->batch;
    {
        std::lock_guard<std::mutex> lk(ps->pool->mu);
        MYNN_REQUIRE((int)ps->pool->free_list.size() >= take, MYNN_ERR_NO_PAGES,
                     "kv_pages_reserve: %d pages wanted, %d free in the pool of %d", take, (int)ps->pool->free_list.size(),
                     ps->pool->n_pages);
        for (int slot = ps->mapped; slot < need; slot++)
            for (int b = 0; b < ps->batch; b++) {
                ps->host[(size_t)b * ps->pages_per_seq + slot] = ps->pool->free_list.back();
                ps->pool->free_list.pop_back();
            }
    }
    // (synchronous: no launch of an executor of this set is in flight when its step reserves)
    hipError_t e = hipMemcpy(ps->dev, ps->host.data(), ps->host.size() * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        // give the pages back: the device table still shows the old mapping
        std::lock_guard<std::mutex> lk(ps->pool->mu);
        for (int slot = ps->mapped; slot < need; slot++)
            for (int b = 0; b < ps->batch; b++) {
                int32_t &pg = ps->host[(size_t)b * ps->pages_per_seq + slot];
                ps->pool->free_list.push_back(pg);
                pg = -1;
            }
        return hip_fail(e, "kv_pages_reserve: table upload");
    }
    ps->mapped = need;
    return 0;
}

KvPaging kv_pages_paging(const mynn_kv_pages *ps) {
    KvPaging pg;
    if (ps) {
        pg.table = ps->dev;
        pg.shift = ps->shift;
        pg.pages_per_seq = ps->pages_per_seq;
    }
    return pg;
}
int kv_pages_batch(const mynn_kv_pages *ps) { return ps ? ps->batch : 0; }
int kv_pages_pool_pages(const mynn_kv_pages *ps) { return ps ? ps->pool->n_pages : 0; }

}  // namespace mynn

extern "C" mynn_kv_pool *mynn_kv_pool_create(int n_pages, int page_rows) {
    if (n_pages <= 0 || page_rows < 32 || page_rows > (1 << 20) || (page_rows & (page_rows - 1))) {
        fail(MYNN_ERR_INVALID, "kv_pool_create: %d pages of %d rows (rows per page: a power of two, 32 or more)", n_pages, page_rows);
        return nullptr;
    }
    mynn_kv_pool *p = new mynn_kv_pool();
    p->n_pages = n_pages;
    p->page_rows = page_rows;
    p->free_list.resize(n_pages);
    for (int i = 0; i < n_pages; i++) p->free_list[i] = n_pages - 1 - i;
    return p;
}

extern "C" int mynn_kv_pool_free_pages(const mynn_kv_pool *pool) {
    MYNN_REQUIRE(pool, MYNN_ERR_INVALID, "kv_pool_free_pages: null pool");
    std::lock_guard<std::mutex> lk(const_cast<mynn_kv_pool *>(pool)->mu);
    return (int)pool->free_list.size();
}

extern "C" int mynn_kv_pool_destroy(mynn_kv_pool *pool) {
    if (!pool) return 0;
    MYNN_REQUIRE(pool->sets == 0, MYNN_ERR_STATE, "kv_pool_destroy: %d page sets still use the pool", pool->sets);
    delete pool;
    return 0;
}

extern "C" mynn_kv_pages *mynn_kv_pages_create(mynn_kv_pool *pool, int batch, int max_seq) {
    if (!pool || batch <= 0 || max_seq <= 0 || max_seq % pool->page_rows) {
        fail(MYNN_ERR_INVALID, "kv_pages_create: batch %d, max_seq %d (a positive multiple of the pool's %d rows per page)", batch,
             max_seq, pool ? pool->page_rows : 0);
        return nullptr;
    }
    mynn_kv_pages *ps = new mynn_kv_pages();
    ps->pool = pool;
    ps->batch = batch;
    ps->pages_per_seq = max_seq / pool->page_rows;
    while ((1 << ps->shift) < pool->page_rows) ps->shift++;
    ps->host.assign((size_t)batch * ps->pages_per_seq, -1);
    hipError_t e = hipMalloc((void **)&ps->dev, ps->host.size() * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemcpy(ps->dev, ps->host.data(), ps->host.size() * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        hip_fail(e, "kv_pages_create");
        if (ps->dev) (void)hipFree(ps->dev);
        delete ps;
        return nullptr;
    }
    std::lock_guard<std::mutex> lk(pool->mu);
    pool->sets++;
    return ps;
}

extern "C" int mynn_kv_pages_reserve(mynn_kv_pages *pages, int64_t rows) { return kv_pages_reserve(pages, (long)rows); }

extern "C" int mynn_kv_pages_release(mynn_kv_pages *ps) {
    MYNN_REQUIRE(ps, MYNN_ERR_INVALID, "kv_pages_release: null page set");
    {
        std::lock_guard<std::mutex> lk(ps->pool->mu);
        // slots in falling order, so that a set that is filled again right away gets its pages back in the same order
        for (int slot = ps->mapped - 1; slot >= 0; slot--)
            for (int b = ps->batch - 1; b >= 0; b--) {
                int32_t &pg = ps->host[(size_t)b * ps->pages_per_seq + slot];
                ps->pool->free_list.push_back(pg);
                pg = -1;
            }
    }
    ps->mapped = 0;
    MYNN_HIP(hipMemcpy(ps->dev, ps->host.data(), ps->host.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    return 0;
}

extern "C" int mynn_kv_pages_mapped_rows(const mynn_kv_pages *ps) { return ps ? ps->mapped << ps->shift : 0; }
extern "C" int mynn_kv_pages_per_seq(const mynn_kv_pages *ps) { return ps ? ps->pages_per_seq : 0; }
extern "C" const int32_t *mynn_kv_pages_table(const mynn_kv_pages *ps) { return ps ? ps->dev : nullptr; }
extern "C" int mynn_kv_pages_table_host(const mynn_kv_pages *ps, int32_t *out) {
    MYNN_REQUIRE(ps && out, MYNN_ERR_INVALID, "kv_pages_table_host: null argument");
    memcpy(out, ps->host.data(), ps->host.size() * sizeof(int32_t));
    return 0;
}

extern "C" int mynn_kv_pages_destroy(mynn_kv_pages *ps) {
    if (!ps) return 0;
    int rc = mynn_kv_pages_release(ps);
    (void)hipFree(ps->dev);
    {
        std::lock_guard<std::mutex> lk(ps->pool->mu);
        ps->pool->sets--;
    }
    delete ps;
    return rc;
}
