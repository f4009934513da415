// LZ4 block codec (host code only; no kernel in this file).
//
// BIDMach stores model checkpoints as `modelmat%02d.lz4` (src/main/scala/BIDMach/models/
// Model.scala:259-262, :284-292 of the reference) and its word2vec input as `.imat.lz4` files;
// the codec behind them is BIDMat's, through the lz4-java library, neither of which is in the
// reference tree.  This is an independent implementation of the published LZ4 block format:
//   a block is a series of sequences; a sequence is a token byte (high nibble: number of literals,
//   low nibble: match length - 4; a nibble of 15 is continued by bytes that are added until one is
//   below 255), the literals, a two-byte little-endian match offset (1..65535, counted back from
//   the current output position) and the optional match-length continuation; the last sequence
//   ends after its literals.  A conforming encoder ends a block with at least 5 literals and does
//   not start a match within the last 12 bytes.
// The stream framing around the blocks is done by the caller (bidmach_amd/matio.py).
#include "../../include/bidmach_w2v.h"

#include <cstdint>
#include <cstring>

namespace {

constexpr int kMinMatch = 4;
constexpr int kLastLiterals = 5;
constexpr int kMatchSafeguard = 12;
constexpr int kHashBits = 14;
constexpr uint32_t kMaxOffset = 65535;

inline uint32_t read32(const uint8_t* p) {
  uint32_t v;
  std::memcpy(&v, p, 4);
  return v;
}

inline uint32_t hash4(uint32_t v) { return (v * 2654435761u) >> (32 - kHashBits); }

// Writes `len` as the continuation of a nibble that already holds 15.
inline bool put_length(uint8_t*& op, const uint8_t* oend, size_t len) {
  while (len >= 255) {
    if (op >= oend) return false;
    *op++ = 255;
    len -= 255;
  }
  if (op >= oend) return false;
  *op++ = (uint8_t)len;
  return true;
}

bool emit_sequence(uint8_t*& op, const uint8_t* oend, const uint8_t* lit, size_t nlit,
                   bool has_match, uint32_t offset, size_t mlen) {
  if (op >= oend) return false;
  uint8_t* token = op++;
  const size_t lcode = nlit >= 15 ? 15 : nlit;
  size_t mcode = 0;
  if (has_match) mcode = (mlen - kMinMatch) >= 15 ? 15 : (mlen - kMinMatch);
  *token = (uint8_t)((lcode << 4) | mcode);
  if (lcode == 15 && !put_length(op, oend, nlit - 15)) return false;
  if ((size_t)(oend - op) < nlit) return false;
  std::memcpy(op, lit, nlit);
  op += nlit;
  if (!has_match) return true;
  if (oend - op < 2) return false;
  *op++ = (uint8_t)(offset & 0xff);
  *op++ = (uint8_t)(offset >> 8);
  if (mcode == 15 && !put_length(op, oend, mlen - kMinMatch - 15)) return false;
  return true;
}

}  // namespace

extern "C" {

size_t w2v_lz4_compress_bound(size_t n) { return n + n / 255 + 16; }

long long w2v_lz4_compress(const void* src_, size_t n, void* dst_, size_t cap) {
  if ((!src_ && n) || !dst_ || n > 0x7fffffffu) return -1;
  const uint8_t* const src = static_cast<const uint8_t*>(src_);
  uint8_t* const dst = static_cast<uint8_t*>(dst_);
  uint8_t* op = dst;
  const uint8_t* const oend = dst + cap;
  const uint8_t* const iend = src + n;
  const uint8_t* anchor = src;

  if (n >= (size_t)kMatchSafeguard + 1) {
    int32_t table[1 << kHashBits];  // last position seen for each hash, 64 KB on the stack
    for (int i = 0; i < (1 << kHashBits); ++i) table[i] = -1;
    const uint8_t* const mflimit = iend - kMatchSafeguard;   // last position a match may start at
    const uint8_t* const matchlimit = iend - kLastLiterals;  // a match may not run past this
    const uint8_t* ip = src;
    while (ip <= mflimit) {
      const uint32_t h = hash4(read32(ip));
      const int32_t cand = table[h];
      table[h] = (int32_t)(ip - src);
      if (cand >= 0 && (size_t)((ip - src) - cand) <= kMaxOffset &&
          read32(src + cand) == read32(ip)) {
        const uint8_t* ref = src + cand;
        size_t mlen = kMinMatch;
        while (ip + mlen < matchlimit && ip[mlen] == ref[mlen]) ++mlen;
        if (!emit_sequence(op, oend, anchor, (size_t)(ip - anchor), true, (uint32_t)(ip - ref),
                           mlen))
          return -1;
        ip += mlen;
        anchor = ip;
      } else {
        ++ip;
      }
    }
  }
  if (!emit_sequence(op, oend, anchor, (size_t)(iend - anchor), false, 0, 0)) return -1;
  return (long long)(op - dst);
}

long long w2v_lz4_decompress(const void* src_, size_t n, void* dst_, size_t cap) {
  if (!src_ || (!dst_ && cap)) return -1;
  const uint8_t* ip = static_cast<const uint8_t*>(src_);
  const uint8_t* const iend = ip + n;
  uint8_t* const dst = static_cast<uint8_t*>(dst_);
  uint8_t* op = dst;
  uint8_t* const oend = dst + cap;
  if (n == 0) return -1;
  for (;;) {
    if (ip >= iend) return -1;
    const unsigned token = *ip++;
    size_t nlit = token >> 4;
    if (nlit == 15) {
      unsigned b;
      do {
        if (ip >= iend) return -1;
        b = *ip++;
        nlit += b;
      } while (b == 255);
    }
    if ((size_t)(iend - ip) < nlit || (size_t)(oend - op) < nlit) return -1;
    std::memcpy(op, ip, nlit);
    ip += nlit;
    op += nlit;
    if (ip == iend) break;  // the last sequence has no match
    if (iend - ip < 2) return -1;
    const size_t offset = (size_t)ip[0] | ((size_t)ip[1] << 8);
    ip += 2;
    if (offset == 0 || offset > (size_t)(op - dst)) return -1;
    size_t mlen = token & 15;
    if (mlen == 15) {
      unsigned b;
      do {
        if (ip >= iend) return -1;
        b = *ip++;
        mlen += b;
      } while (b == 255);
    }
    mlen += kMinMatch;
    if ((size_t)(oend - op) < mlen) return -1;
    const uint8_t* ref = op - offset;
    for (size_t k = 0; k < mlen; ++k) op[k] = ref[k];  // byte by byte: the ranges may overlap
    op += mlen;
  }
  return (long long)(op - dst);
}

}  // extern "C"
