// Host-side check of the LDS tile layout the fast kernels share (compiled for the host only and run
// on the CPU by tests/test_lds_layout.py).  For every padded head dimension it walks all lanes, waves
// and wave-loads of a 64-row tile and verifies that
//   * the slot an LDS-direct load writes is where the fragment readers (swz_off) look for the chunk
//     the loader fetched into it, and every (row, chunk) of the tile is written exactly once;
//   * the loader's shortcut holds: the chunk does not depend on the load index, except with rows of
//     256 halves, where odd loads take the even load's chunk with bit 1 flipped;
//   * both read patterns are free of bank conflicts on 64 banks of 4 bytes: 16 consecutive rows at
//     one logical chunk (ds_read_b128) and 4 consecutive rows x 4 consecutive chunks (transposing read).
#include <cstdio>
#include <set>
#include <vector>

#include "fa2_common.hpp"

template <int DP>
int check() {
  constexpr int ROWS = 64, NW = 4;
  using TL = TileLoader<DP, ROWS, NW, false>;
  constexpr int LP = TL::LP, CPR = TL::CPR, RPL = TL::RPL;
  int bad = 0;
  std::vector<int> seen(ROWS * CPR, 0);
  for (int i = 0; i < TL::LOADS; i++)
    for (int wave = 0; wave < NW; wave++)
      for (int lane = 0; lane < 64; lane++) {
        const int row = i * NW * RPL + wave * RPL + lane / CPR;
        const int chunk = TL::chunk_of(lane, wave, i);
        const int written = ((i * NW + wave) * 1024 + 16 * lane) / 2;  // element offset of the slot
        if (row >= ROWS || chunk < 0 || chunk >= CPR) { bad++; continue; }
        if (written != swz_off<LP>(row, chunk)) bad++;
        seen[row * CPR + chunk]++;
        const int c0 = TL::chunk_of(lane, wave, 0);
        if (chunk != ((TL::BY_PARITY && (i & 1)) ? (c0 ^ 2) : c0)) bad++;
      }
  for (int v : seen) bad += v != 1;
  auto banks_distinct = [&](const std::vector<int> &slot_offsets) {  // 16-byte slots, element offsets
    std::set<int> banks;
    for (int off : slot_offsets)
      for (int w = 0; w < 4; w++) banks.insert(((off * 2) / 4 + w) % 64);
    return banks.size() == slot_offsets.size() * 4;
  };
  for (int r0 = 0; r0 < ROWS; r0 += 16)
    for (int c = 0; c < CPR; c++) {
      std::vector<int> offs;
      for (int j = 0; j < 16; j++) offs.push_back(swz_off<LP>(r0 + j, c));
      bad += !banks_distinct(offs);
    }
  for (int r0 = 0; r0 < ROWS; r0 += 4)
    for (int c0 = 0; c0 + 4 <= CPR; c0 += 4) {
      std::vector<int> offs;
      for (int j = 0; j < 4; j++)
        for (int c = 0; c < 4; c++) offs.push_back(swz_off<LP>(r0 + j, c0 + c));
      bad += !banks_distinct(offs);
    }
  printf("DP %3d: row pitch %3d, %2d slots per row, %d wave-loads per wave, by parity %d: %s\n", DP, LP, CPR, TL::LOADS,
         (int)TL::BY_PARITY, bad ? "FAILED" : "ok");
  return bad;
}

int main() {
  int bad = 0;
  bad += check<32>();
  bad += check<64>();
  bad += check<96>();
  bad += check<128>();
  bad += check<192>();
  bad += check<256>();
  return bad ? 1 : 0;
}
