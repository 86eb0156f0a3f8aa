// Host-side check of index arithmetic the kernels and launchers share (compiled for the host only and
// run on the CPU by tests/test_lds_layout.py): the workgroup -> (head, tile) mapping with its head
// groups, and the LDS tile layout.  For every padded head dimension it walks all lanes, waves and
// wave-loads of a 64-row tile and verifies that
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
#include "fa2_launch.hpp"

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

// Workgroup index -> (head, tile rank) with the head groups the launchers compute: every pair is
// visited exactly once, ranks never decrease inside a group (heaviest tile first), group sizes are
// multiples of 8, and with a head count that is a multiple of 8 all workgroups of a head have the
// same index modulo 8, that is, land on one XCD.
int check_mapping() {
  int bad = 0, cases = 0;
  for (int table_group : {32, 64})
    for (int heads : {1, 3, 8, 16, 24, 33, 48, 63, 64, 72, 80, 96, 100, 128, 129, 192, 2048})
      for (int tiles : {1, 2, 7, 32}) {
        const int group = fa2::equal_head_groups(table_group, heads);
        if (group % 8 != 0 || group < 8) bad++;
        if (heads >= 2 * table_group && group > 2 * table_group) bad++;  // groups stay near the table's size
        std::vector<int> seen(heads * tiles, 0), xcd(heads, -1);
        int last_rank = 0, last_group = -1;
        for (int i = 0; i < heads * tiles; i++) {
          int bh = -1, rank = -1;
          fa2::map_workgroup(i, heads, tiles, group, bh, rank);
          if (bh < 0 || bh >= heads || rank < 0 || rank >= tiles) { bad++; continue; }
          seen[bh * tiles + rank]++;
          const int g = bh / group;
          if (g == last_group && rank < last_rank) bad++;
          if (g < last_group) bad++;  // groups are walked in order
          last_group = g;
          last_rank = rank;
          if (heads % 8 == 0) {
            if (xcd[bh] < 0) xcd[bh] = i % 8;
            else if (xcd[bh] != i % 8) bad++;
          }
        }
        for (int v : seen) bad += v != 1;
        cases++;
      }
  printf("workgroup mapping, %d cases: %s\n", cases, bad ? "FAILED" : "ok");
  return bad;
}

int main() {
  int bad = check_mapping();
  bad += check<32>();
  bad += check<64>();
  bad += check<96>();
  bad += check<128>();
  bad += check<192>();
  bad += check<256>();
  return bad ? 1 : 0;
}
