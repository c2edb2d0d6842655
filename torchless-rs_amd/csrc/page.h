// Positions in a page of the cache: the one place where the number is written.
// The kernels (common.hpp), the host library's books (host/books.cpp) and the
// Python side (kernels/page.py reads this file) all take it from here, and each
// library reports what it was compiled with (tl_page_size, tl_host_page) so that
// a mismatch is refused when a library is loaded.  The attention kernels lay a
// page's keys and values out for the matrix cores in tiles of 64 positions, so
// another value needs those kernels changed, not only this line.
#pragma once
#define TL_PAGE 64
