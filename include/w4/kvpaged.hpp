#pragma once

// Paged W4 KV cache, host side.  Same API and error behaviour as the
// reference's include/w4/kvpaged.hpp (cited per function).
//
// Every head owns a pool slab of npages * page rows in the W4 cache row format;
// a block table maps logical page i of the sequence to a physical page, so
// logical position t lives at pool row block_table[t / page] * page + t % page.
// Paging moves rows, it never changes them: sequences whose tables name the
// same physical pages share that prefix once.

#include <hip/hip_fp16.h>

#include <stdexcept>
#include <vector>

#include "kvcache.hpp"

namespace w4::kv {

// kvpaged.hpp:25-34
struct KVCacheW4Paged {
  int H = 0, S = 0, D = 0, gs = 0, G = 0;
  int page = 0;
  int npages = 0;
  bool symmetric = true;
  std::vector<uint32_t> q_k, q_v;
  std::vector<__half> s_k, s_v;
  std::vector<uint32_t> z_k, z_v;
  std::vector<int> block_table;
};

namespace detail {

// true when `bt` names each of its pages once and stays below `limit`
inline bool table_is_injective(const std::vector<int>& bt, int limit) {
  std::vector<char> used((size_t)std::max(limit, 0), 0);
  for (const int b : bt) {
    if (b < 0 || b >= limit || used[(size_t)b]) return false;
    used[(size_t)b] = 1;
  }
  return true;
}

}  // namespace detail

// kvpaged.hpp:36-67
inline void validate_paged(const KVCacheW4Paged& c) {
  using w4::detail::require;
  require(c.H >= 1 && c.S >= 1 && c.D >= 1, "paged: bad dims");
  require(c.gs >= 8 && c.gs % 8 == 0, "paged: gs must be a multiple of 8");
  require(c.G == (c.D + c.gs - 1) / c.gs, "paged: G inconsistent with D, gs");
  require(c.page >= 1 && c.npages >= 1, "paged: bad page geometry");
  const size_t logical_pages = ((size_t)c.S + c.page - 1) / c.page;
  require(c.block_table.size() == logical_pages, "paged: block table size");
  require((size_t)c.npages >= logical_pages, "paged: pool smaller than table");
  const size_t rows = (size_t)c.H * c.npages * c.page;
  require(c.q_k.size() == rows * words(c.D) && c.q_v.size() == rows * words(c.D), "paged: q size");
  require(c.s_k.size() == rows * c.G && c.s_v.size() == rows * c.G, "paged: scales size");
  require(c.symmetric || (c.z_k.size() == rows * words(c.G) && c.z_v.size() == rows * words(c.G)),
          "paged: zeros size");
  for (const int b : c.block_table)
    require(b >= 0 && b < c.npages, "paged: block table entry out of pool");
  require(detail::table_is_injective(c.block_table, c.npages), "paged: block table repeats a page");
}

// Scatter a contiguous cache into a pool of exactly bt.size() pages
// (kvpaged.hpp:72-134); rows past S in the last page stay zero.
inline KVCacheW4Paged paged_from_contiguous(const KVCacheW4& c, int page,
                                            const std::vector<int>& bt) {
  using w4::detail::require;
  validate_cache(c);
  require(page >= 1, "paged_from: bad page size");
  require(bt.size() == ((size_t)c.S + (size_t)page - 1) / (size_t)page,
          "paged_from: block table size");
  require(detail::table_is_injective(bt, (int)bt.size()), "paged_from: bad block table");
  KVCacheW4Paged p;
  p.H = c.H;
  p.S = c.S;
  p.D = c.D;
  p.gs = c.gs;
  p.G = c.G;
  p.page = page;
  p.npages = (int)bt.size();
  p.symmetric = c.symmetric;
  p.block_table = bt;
  const size_t pool_rows = (size_t)p.npages * page;
  auto scatter = [&](const auto& src, auto& dst, size_t per_row, auto fill) {
    dst.assign((size_t)c.H * pool_rows * per_row, fill);
    for (int h = 0; h < c.H; ++h)
      for (int t = 0; t < c.S; ++t) {
        const size_t row = (size_t)bt[(size_t)(t / page)] * page + (size_t)(t % page);
        std::copy_n(src.begin() + ((size_t)h * c.S + t) * per_row, per_row,
                    dst.begin() + ((size_t)h * pool_rows + row) * per_row);
      }
  };
  scatter(c.q_k, p.q_k, (size_t)words(c.D), 0u);
  scatter(c.q_v, p.q_v, (size_t)words(c.D), 0u);
  scatter(c.s_k, p.s_k, (size_t)c.G, __float2half_rn(0.0f));
  scatter(c.s_v, p.s_v, (size_t)c.G, __float2half_rn(0.0f));
  if (!c.symmetric) {
    scatter(c.z_k, p.z_k, (size_t)words(c.G), 0u);
    scatter(c.z_v, p.z_v, (size_t)words(c.G), 0u);
  }
  return p;
}

}  // namespace w4::kv
