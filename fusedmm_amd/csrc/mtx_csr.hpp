// MatrixMarket coordinate text -> CSR, in the order the reference's loader
// produces (test/include/IO.h:62-162 ReadASCII, CSC.h:147-189, CSR.h:154-186).
//
// Rules restated from that code:
//  - leading lines that start with '%' are skipped; if any of them contains
//    the word "symmetric" every off-diagonal entry is mirrored and diagonal
//    entries are dropped (IO.h:70-79, 127-143); otherwise self-loops stay;
//  - the size line is "rows cols entries"; at most that many entry lines are read;
//  - an entry is "row col [value]", single-space separated, 1-based; the value
//    is read with atoi (fractions truncate toward zero), 1.0 when absent (IO.h:106-124);
//  - the reference goes COO -> CSC (stable counting sort by column, then
//    std::sort of (row, value) pairs inside each column) -> CSR (columns scanned
//    in ascending order), so inside a CSR row column ids ascend, duplicates are
//    kept, and duplicates of one (row, col) are ordered by value.  Sorting the
//    triples by (row, col, value) gives the same arrays and is what is done here.
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace fmm_host {

template <typename IT>
struct CsrMatrix {
   IT rows = 0, cols = 0, nnz = 0;
   std::vector<IT> rowptr;      // rows + 1
   std::vector<IT> colids;      // nnz, ascending inside a row
   std::vector<float> values;   // nnz
};

struct Entry {
   int64_t row, col;
   float val;
};

// Returns an empty string on success, else what went wrong.
template <typename IT>
std::string load_mtx(const char *path, CsrMatrix<IT> &out)
{
   FILE *f = std::fopen(path, "rb");
   if (!f) return std::string("cannot open ") + path;
   std::fseek(f, 0, SEEK_END);
   long sz = std::ftell(f);
   std::fseek(f, 0, SEEK_SET);
   std::string text((size_t)sz, '\0');
   if (sz > 0 && std::fread(&text[0], 1, (size_t)sz, f) != (size_t)sz)
   {
      std::fclose(f);
      return "short read";
   }
   std::fclose(f);

   const char *p = text.c_str(), *end = p + text.size();
   auto next_line = [&](const char *&b, const char *&e) -> bool {
      if (p >= end) return false;
      b = p;
      const char *nl = (const char *)std::memchr(p, '\n', (size_t)(end - p));
      e = nl ? nl : end;
      p = nl ? nl + 1 : end;
      return true;
   };
   bool symmetric = false;
   const char *b, *e;
   // header / comment lines
   while (p < end && *p == '%')
   {
      next_line(b, e);
      if (std::string(b, e).find("symmetric") != std::string::npos) symmetric = true;
   }
   if (!next_line(b, e)) return "missing size line";
   long long m = 0, n = 0, declared = 0;
   if (std::sscanf(std::string(b, e).c_str(), "%lld %lld %lld", &m, &n, &declared) != 3) return "bad size line";

   std::vector<Entry> tr;
   tr.reserve((size_t)(symmetric ? 2 * declared : declared));
   long long read = 0;
   while (read < declared && next_line(b, e))
   {
      std::string line(b, e);
      const char *ch = line.c_str();
      Entry t;
      t.row = std::atoi(ch) - 1;
      const char *sp = std::strchr(ch, ' ');
      if (!sp) break;                       // the reference would dereference NULL here
      t.col = std::atoi(sp + 1) - 1;
      sp = std::strchr(sp + 1, ' ');
      t.val = sp ? (float)std::atoi(sp + 1) : 1.0f;
      read++;
      if (symmetric)
      {
         if (t.row == t.col) continue;      // diagonal dropped
         tr.push_back(t);
         tr.push_back(Entry{t.col, t.row, t.val});
      }
      else
         tr.push_back(t);
   }
   for (const Entry &t : tr)
      if (t.row < 0 || t.row >= m || t.col < 0 || t.col >= n) return "entry outside the declared shape";

   std::sort(tr.begin(), tr.end(), [](const Entry &a, const Entry &c) {
      if (a.row != c.row) return a.row < c.row;
      if (a.col != c.col) return a.col < c.col;
      return a.val < c.val;
   });
   out.rows = (IT)m;
   out.cols = (IT)n;
   out.nnz = (IT)tr.size();
   out.rowptr.assign((size_t)m + 1, 0);
   out.colids.resize(tr.size());
   out.values.resize(tr.size());
   for (size_t i = 0; i < tr.size(); i++)
   {
      out.rowptr[(size_t)tr[i].row + 1]++;
      out.colids[i] = (IT)tr[i].col;
      out.values[i] = tr[i].val;
   }
   for (size_t r = 0; r < (size_t)m; r++) out.rowptr[r + 1] += out.rowptr[r];
   return "";
}

}  // namespace fmm_host
