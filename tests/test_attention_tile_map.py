"""The scalar helpers with which the attention kernels walk the visible-tile map of a mask tensor
(anygpu_amd/csrc/attention_tile_map.hpp): the next set tile of a range, and the share of a part among the set tiles.
Their text is compiled for the host (they use nothing of the device but its qualifiers) and checked against brute
force over random maps, ranges and part counts.  CPU only."""
import subprocess
from pathlib import Path

REPO = Path(__file__).resolve().parent.parent

HARNESS = r"""
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>
#define __device__
#define __forceinline__ inline
#define __restrict__
%s
int main()
{
	std::mt19937_64 rng(1);
	long checks = 0;
	for (int iter = 0; iter < 20000; ++iter)
	{
		const int tiles = 1 + rng() %% 300, words = (tiles + 63) / 64;
		std::vector<unsigned long long> map(words, 0);
		const int density = rng() %% 5;                          // 0: nothing set, 4: everything
		for (int t = 0; t < tiles; ++t)
			if (density == 4 || (density > 0 && (int)(rng() %% 4) < density)) map[t >> 6] |= 1ull << (t & 63);
		int a = rng() %% tiles, b = rng() %% tiles;
		int t0 = std::min(a, b), t1 = std::max(a, b);
		if (rng() %% 10 == 0) t0 = 0, t1 = tiles - 1;
		std::vector<int> set;
		for (int t = t0; t <= t1; ++t)
			if (map[t >> 6] >> (t & 63) & 1) set.push_back(t);
		for (int t = t0; t <= t1 + 1; ++t, ++checks)
		{
			int want = t1 + 1;
			for (int v : set)
				if (v >= t) { want = v; break; }
			if (anygpu_next(map.data(), t, t1) != want) { std::printf("next set tile: mismatch\n"); return 1; }
		}
		const int parts = 1 + rng() %% 9, total = (int)set.size(), per = (total + parts - 1) / parts;
		for (int p = 0; p < parts; ++p, ++checks)
		{
			int first = t0, last = t1;
			anygpu_share(map.data(), p, parts, first, last);
			const int lo = p * per, hi = std::min(lo + per, total);
			if (per == 0 || lo >= hi)
			{
				if (first <= last) { std::printf("share: expected an empty one\n"); return 1; }
				continue;
			}
			if (first != set[lo] || last != set[hi - 1]) { std::printf("share: mismatch\n"); return 1; }
		}
	}
	std::printf("ok %%ld\n", checks);
	return 0;
}
"""


def test_tile_map_helpers_against_brute_force(tmp_path):
    text = (REPO / "anygpu_amd" / "csrc" / "attention_tile_map.hpp").read_text()
    begin = text.index("__device__ __forceinline__ int attention_next_visible_tile")
    end = text.index("}  // namespace anygpu")
    body = text[begin:end].replace("attention_next_visible_tile", "anygpu_next").replace("attention_visible_share", "anygpu_share")
    src = tmp_path / "tile_map_check.cpp"
    src.write_text(HARNESS % body)
    exe = tmp_path / "tile_map_check"
    subprocess.run(["g++", "-O1", "-std=c++17", "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert out.startswith("ok "), out
