// Host-side bounds model of the hot kernels' fetch patterns (plain g++, no GPU): runs the address
// arithmetic of litenn_amd/csrc/fetch_model.hpp -- the very functions the kernels call -- for every
// thread of a launch over page-exact, ragged and minimal shapes, and checks
//   * every requested 16-byte piece is 16-byte aligned and holds at least one byte of its tensor
//     (so it lies in a page the tensor occupies);
//   * the pieces a kernel consumes are fetched from the right addresses and cover what it reads;
//   * rows, activation elements and cache rows are each covered, none outside its array.
// It also shows that the checker has teeth: the matrix-core GEMM's piece arithmetic as it was before
// its over-fetch was fixed (no redirection of a piece that holds no byte of its chunk) fails on the
// Q2_K 512 x 512 tensor that once faulted a GPU.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <vector>

#include "../../litenn_amd/csrc/fetch_model.hpp"

namespace fm = litenn_hip::fetch;

static int g_failures = 0;
#define CHECK(cond, ...)                                                                                               \
	do                                                                                                                 \
	{                                                                                                                  \
		if (!(cond))                                                                                                   \
		{                                                                                                              \
			if (++g_failures <= 20)                                                                                    \
			{                                                                                                          \
				std::printf("FAIL %s:%d %s: ", __FILE__, __LINE__, #cond);                                             \
				std::printf(__VA_ARGS__);                                                                              \
				std::printf("\n");                                                                                     \
			}                                                                                                          \
		}                                                                                                              \
	} while (0)

struct Format
{
	const char* name;
	int chunk_bytes;   // bytes of 256 elements
	bool aligned16;    // the GEMM's view: chunks start on 16-byte boundaries
	int base_align;    // what the GEMM launcher demands of the tensor's address
	int stream_slice;  // bytes of 4096 elements (one wavefront's slice in the streaming GEMV)
};
static const Format kFormats[] = {
	{ "Q4_0", 144, true, 16, 2304 }, { "Q4_1", 160, true, 16, 2560 }, { "Q5_0", 176, true, 16, 2816 },
	{ "Q5_1", 192, true, 16, 3072 }, { "Q8_0", 272, true, 16, 4352 }, { "Q4_K", 144, true, 16, 2304 },
	{ "Q5_K", 176, true, 16, 2816 }, { "Q2_K", 84, false, 4, 1344 },  { "Q3_K", 110, false, 2, 1760 },
	{ "Q6_K", 210, false, 2, 3360 },
};

constexpr uintptr_t kPage = 4096;

// ---- matrix-core GEMM weight pieces -------------------------------------------------------------
typedef uintptr_t (*PieceFn)(uintptr_t, int, int, bool, int);

static uintptr_t piece_without_redirection(uintptr_t row_start, int c, int chunk_bytes, bool aligned16, int offset)
{
	const uintptr_t chunk = row_start + static_cast<size_t>(c) * chunk_bytes;
	return (aligned16 ? chunk : (chunk & ~uintptr_t{ 15 })) + offset;
}

// returns the number of pieces that touch no byte of [base, base + bytes)
// base_up != 0: the gated form (ng = 2), whose second weight group holds the same rows of a second
// n-row matrix at base_up
static long gemm_case(const Format& f, int ng, int waves, int n, int chunks, uintptr_t base, PieceFn piece_fn,
                      bool check_contents, uintptr_t base_up = 0)
{
	const bool gated = base_up != 0;
	const size_t row_bytes = static_cast<size_t>(chunks) * f.chunk_bytes;
	const size_t bytes = static_cast<size_t>(n) * row_bytes;
	const int pieces = fm::gemm_weight_pieces(f.chunk_bytes, f.aligned16);
	const int loads = (ng * 16 * pieces + 63) / 64;
	const int bn = gated ? 16 * waves : 16 * waves * ng;
	const auto matrix_of = [&](int slot_row) { return gated && slot_row >= 16 ? base_up : base; };
	const auto row_of = [&](int slot_row) { return gated ? (slot_row & 15) : slot_row; };
	long outside = 0;
	for (int block = 0; block < (n + bn - 1) / bn; ++block)
	{
		for (int wave = 0; wave < waves; ++wave)
		{
			const int n_base = (block * waves + wave) * 16 * (gated ? 1 : ng);
			for (int c = 0; c < chunks; ++c)
			{
				std::map<int, uintptr_t> slot; // slot byte offset of a piece -> where it was fetched from
				for (int i = 0; i < loads; ++i)
				{
					for (int lane = 0; lane < 64; ++lane)
					{
						const fm::GemmWeightRequest rq = fm::gemm_weight_request(i, lane, ng, pieces);
						if (!(64 * (i + 1) <= ng * 16 * pieces || rq.issued))
						{
							continue;
						}
						CHECK(rq.row >= 0 && rq.row < 16 * ng && rq.offset >= 0 && rq.offset < 16 * pieces, "%s row %d off %d",
						      f.name, rq.row, rq.offset);
						const uintptr_t mbase = matrix_of(rq.row), end = mbase + bytes;
						const uintptr_t row_start =
						    mbase + static_cast<size_t>(fm::gemm_weight_row(n_base, row_of(rq.row), n)) * row_bytes;
						const uintptr_t from = piece_fn(row_start, c, f.chunk_bytes, f.aligned16, rq.offset);
						if (check_contents)
						{
							CHECK(from % 16 == 0, "%s n %d: piece at %#zx is not aligned", f.name, n, static_cast<size_t>(from));
						}
						if (!(from < end && from + 16 > mbase))
						{
							++outside;
						}
						// the i-th instruction writes 1 KB of the slot: lane l at 1024 i + 16 l
						slot[1024 * i + 16 * lane] = from;
					}
				}
				if (!check_contents)
				{
					continue;
				}
				// what the decoders read: row r of the wavefront at slot offset r * 16 pieces + mis,
				// chunk_bytes bytes, which must be the chunk's own bytes
				for (int r = 0; r < 16 * ng; ++r)
				{
					const uintptr_t row_start =
					    matrix_of(r) + static_cast<size_t>(fm::gemm_weight_row(n_base, row_of(r), n)) * row_bytes;
					const uintptr_t chunk = row_start + static_cast<size_t>(c) * f.chunk_bytes;
					const int mis = fm::gemm_weight_misalignment(row_start, c, f.chunk_bytes, f.aligned16);
					for (int b = 0; b < f.chunk_bytes; ++b)
					{
						const int at = r * 16 * pieces + mis + b;
						const auto it = slot.find(at & ~15);
						CHECK(it != slot.end() && it->second + (at & 15) == chunk + b, "%s n %d chunk %d row %d byte %d", f.name, n, c,
						      r, b);
					}
				}
			}
		}
	}
	return outside;
}

static void test_gemm_weight_pieces()
{
	const int tiles[][2] = { { 2, 8 }, { 1, 8 }, { 1, 4 } }; // weight groups per wavefront, wavefronts
	long cases = 0;
	for (const Format& f : kFormats)
	{
		for (const auto& t : tiles)
		{
			for (int n : { 1, 15, 16, 17, 33, 128, 129, 512 })
			{
				for (int chunks : { 1, 2, 3, 8 })
				{
					const size_t bytes = static_cast<size_t>(n) * chunks * f.chunk_bytes;
					std::vector<uintptr_t> bases;
					for (int mis = 0; mis < 16; mis += f.base_align)
					{
						bases.push_back(64 * kPage + mis); // every misalignment the launcher accepts
					}
					const uintptr_t ends_on_page = 1024 * kPage - bytes; // the tensor's last byte is a page's last
					if (ends_on_page % f.base_align == 0)
					{
						bases.push_back(ends_on_page);
					}
					for (uintptr_t base : bases)
					{
						const long outside = gemm_case(f, t[0], t[1], n, chunks, base, fm::gemm_weight_piece, true);
						CHECK(outside == 0, "%s ng %d waves %d n %d chunks %d base %#zx: %ld pieces outside the tensor", f.name, t[0],
						      t[1], n, chunks, static_cast<size_t>(base), outside);
						++cases;
						// the gated form: the gate matrix at `base`, the up matrix ending on a page far behind it
						const uintptr_t up = 4096 * kPage - bytes;
						if (t[0] == 2 && up % f.base_align == 0)
						{
							const long out2 = gemm_case(f, 2, t[1], n, chunks, base, fm::gemm_weight_piece, true, up);
							CHECK(out2 == 0, "%s gated n %d chunks %d base %#zx: %ld pieces outside their matrix", f.name, n, chunks,
							      static_cast<size_t>(base), out2);
							++cases;
						}
					}
				}
			}
		}
	}
	std::printf("gemm weight pieces: %ld launches walked\n", cases);
	// the arithmetic as it was before the fix, on the tensor that faulted: Q2_K, 512 rows of 512
	// elements = 21 pages exactly; the last piece of the last rows' last chunk lies in the next page
	const Format& q2k = kFormats[7];
	const size_t bytes = 512 * 2 * 84;
	CHECK(bytes == 21 * kPage, "Q2_K 512 x 512 is 21 pages");
	const long before = gemm_case(q2k, 1, 4, 512, 2, 512 * kPage, piece_without_redirection, false);
	const long after = gemm_case(q2k, 1, 4, 512, 2, 512 * kPage, fm::gemm_weight_piece, false);
	CHECK(before > 0, "the pre-fix arithmetic must be caught");
	CHECK(after == 0, "the current arithmetic stays inside");
	std::printf("Q2_K 512 x 512, page-exact: %ld pieces behind the tensor before the fix, %ld now\n", before, after);
}

// ---- streaming GEMM for few activation rows -----------------------------------------------------
// A workgroup owns a run of consecutive rows and walks it in tiles of 16; wavefront w of eight or sixteen fetches
// the bytes of chunks [w cpw, (w + 1) cpw) of every row of a tile (its slice) with the matrix-core
// GEMM's piece arithmetic, the slice in the place of a chunk.
static void test_gemm_stream_pieces()
{
	long cases = 0;
	for (const Format& f : kFormats)
	{
		for (int geometry : { 801, 802, 804, 1601, 1602 }) // wavefronts x 100 + chunks per wavefront
		{
			const int waves = geometry / 100, cpw = geometry % 100;
			const int slice_bytes = cpw * f.chunk_bytes;
			const size_t row_bytes = static_cast<size_t>(waves) * slice_bytes;
			const int pieces = fm::gemm_weight_pieces(slice_bytes, f.aligned16);
			const int loads = (16 * pieces + 63) / 64;
			for (int n : { 1, 15, 16, 17, 56, 57, 100, 300 })
			{
				for (int cus : { 256, 8, 1 })
				{
					const size_t bytes = static_cast<size_t>(n) * row_bytes;
					std::vector<uintptr_t> bases;
					for (int mis = 0; mis < 16; mis += f.base_align)
					{
						bases.push_back(64 * kPage + mis);
					}
					const uintptr_t ends_on_page = 4096 * kPage - bytes;
					if (ends_on_page % f.base_align == 0)
					{
						bases.push_back(ends_on_page);
					}
					int rows = (n + cus - 1) / cus;
					rows = (rows + 3) / 4 * 4;
					const int blocks = (n + rows - 1) / rows;
					for (uintptr_t base : bases)
					{
						const uintptr_t end = base + bytes;
						std::vector<int> stored(n, 0);
						for (int block = 0; block < blocks; ++block)
						{
							const int row0 = block * rows;
							const int block_rows = rows < n - row0 ? rows : n - row0;
							CHECK(block_rows > 0, "%s n %d: empty workgroup %d", f.name, n, block);
							const int last_row = row0 + block_rows - 1;
							for (int t = 0; t < (block_rows + 15) / 16; ++t)
							{
								for (int wave = 0; wave < waves; ++wave)
								{
									std::vector<uintptr_t> slot(static_cast<size_t>(loads) * 64, 0); // by 16-byte piece of the slot
									for (int i = 0; i < loads; ++i)
									{
										for (int lane = 0; lane < 64; ++lane)
										{
											const fm::GemmWeightRequest rq = fm::gemm_weight_request(i, lane, 1, pieces);
											if (!(64 * (i + 1) <= 16 * pieces || rq.issued))
											{
												continue;
											}
											const int row = fm::gemm_weight_row(row0 + 16 * t, rq.row, last_row + 1);
											CHECK(row >= row0 && row <= last_row, "%s: row %d outside the run", f.name, row);
											const uintptr_t row_start = base + static_cast<size_t>(row) * row_bytes;
											const uintptr_t from = fm::gemm_weight_piece(row_start, wave, slice_bytes, f.aligned16, rq.offset);
											CHECK(from % 16 == 0, "%s: piece not aligned", f.name);
											CHECK(from < end && from + 16 > base, "%s cpw %d n %d base %#zx: piece outside the tensor", f.name, cpw,
											      n, static_cast<size_t>(base));
											slot[64 * i + lane] = from;
										}
									}
									for (int r = 0; r < 16; ++r)
									{
										const int row = fm::gemm_weight_row(row0 + 16 * t, r, last_row + 1);
										const uintptr_t row_start = base + static_cast<size_t>(row) * row_bytes;
										const uintptr_t slice = row_start + static_cast<size_t>(wave) * slice_bytes;
										const int mis = fm::gemm_weight_misalignment(row_start, wave, slice_bytes, f.aligned16);
										for (int b = 0; b < slice_bytes; ++b)
										{
											const int at = r * 16 * pieces + mis + b;
											const uintptr_t from = slot[at >> 4];
											CHECK(from != 0 && from + (at & 15) == slice + b, "%s cpw %d n %d row %d byte %d", f.name,
											      cpw, n, r, b);
										}
										if (wave == 0 && row0 + 16 * t + r <= last_row)
										{
											++stored[row0 + 16 * t + r];
										}
									}
								}
							}
						}
						for (int r = 0; r < n; ++r)
						{
							CHECK(stored[r] == 1, "%s n %d: row %d stored %d times", f.name, n, r, stored[r]);
						}
						++cases;
					}
				}
			}
		}
	}
	std::printf("streaming gemm: %ld launches walked\n", cases);
}

// ---- streaming GEMV ------------------------------------------------------------------------------
static void test_stream_rows_and_pieces()
{
	long cases = 0;
	for (const Format& f : kFormats)
	{
		for (int k : { 256, 512, 1024, 4096, 4352, 8192, 11008, 12288, 14336, 28672, 32768 })
		{
			const uint32_t row_bytes = static_cast<uint32_t>(k / 256 * f.chunk_bytes);
			const int slices = (k + 4095) / 4096;
			if (slices > 8 || row_bytes % 16 != 0)
			{
				continue; // the launcher sends such a shape to the register kernel
			}
			// three-slice rows also run with twelve wavefronts (four groups)
			for (int groups : { 8 / slices, slices == 3 ? 4 : 0 })
			{
			if (groups == 0 || k > 64 * slices * groups * 4 * 8)
			{
				continue; // more than eight 128-bit activation loads per thread: register kernel as well
			}
			const int loads = (f.stream_slice + 1023) / 1024;
			for (int whole = 0; whole < 2; ++whole)
			{
				if (whole && k != 4096)
				{
					continue; // the whole-slice instance exists for K = 4096 only
				}
				std::vector<int> covered(row_bytes, 0);
				for (int s = 0; s < slices; ++s)
				{
					const uint32_t slice_off = static_cast<uint32_t>(s) * f.stream_slice;
					CHECK(slice_off < row_bytes, "%s k %d slice %d starts behind the row", f.name, k, s);
					const uint32_t len = fm::stream_slice_len(whole != 0, f.stream_slice, row_bytes, slice_off);
					CHECK(len >= 16 && len % 16 == 0 && slice_off + len <= row_bytes, "%s k %d slice %d len %u", f.name, k, s, len);
					for (int i = 0; i < loads; ++i)
					{
						for (int lane = 0; lane < 64; ++lane)
						{
							const fm::StreamPiece p = fm::stream_row_piece(i, lane, len, whole != 0);
							if (!p.issued)
							{
								continue;
							}
							CHECK(p.offset + 16 <= len, "%s k %d: piece %u + 16 > %u", f.name, k, p.offset, len);
							if (1024u * i + 16u * lane < len) // a consumed piece sits where the unit reads it
							{
								CHECK(p.offset == 1024u * i + 16u * lane, "%s k %d: piece misplaced", f.name, k);
								for (int b = 0; b < 16; ++b)
								{
									++covered[slice_off + p.offset + b];
								}
							}
						}
					}
				}
				for (uint32_t b = 0; b < row_bytes; ++b)
				{
					CHECK(covered[b] == 1, "%s k %d: row byte %u fetched %d times", f.name, k, b, covered[b]);
				}
				// activations: 128-bit loads, clamped so that every thread issues every one of them
				const int threads = 64 * slices * groups;
				const int per_thread = (k / 4 + threads - 1) / threads;
				const int xp = per_thread <= 2 ? 2 : (per_thread <= 4 ? 4 : 8);
				CHECK(per_thread <= xp, "%s k %d: %d loads per thread", f.name, k, per_thread);
				std::vector<int> x_seen(k, 0);
				for (int tid = 0; tid < threads; ++tid)
				{
					for (int j = 0; j < xp; ++j)
					{
						const int at = fm::stream_x_index(tid, j, threads, k);
						CHECK(at >= 0 && at + 4 <= k && at % 4 == 0, "%s k %d: x load at %d", f.name, k, at);
						if ((tid + j * threads) * 4 < k)
						{
							for (int e = 0; e < 4; ++e)
							{
								++x_seen[at + e];
							}
						}
					}
				}
				for (int e = 0; e < k; ++e)
				{
					CHECK(x_seen[e] == 1, "%s k %d: activation %d staged %d times", f.name, k, e, x_seen[e]);
				}
				// rows: one round of workgroups, every row walked by exactly one wavefront group
				for (int n_total : { 1, 2, 7, 100, 4096, 11008, 32000, 128256 })
				{
					for (int max_blocks : { 256, 64, 1 })
					{
						int rows = (n_total + max_blocks * groups - 1) / (max_blocks * groups);
						rows = rows < 1 ? 1 : (rows > 64 ? 64 : rows);
						// every pair of runs the launcher may choose: the first half of the groups walk `run`
						// rows, the second half `run - diff` (an even number of groups, both at least one row)
						for (int diff = 0; diff < rows && (diff == 0 || groups % 2 == 0); ++diff)
						{
							const int block_rows = fm::stream_block_rows(groups, rows, diff);
							const int blocks = (n_total + block_rows - 1) / block_rows;
							std::vector<int> walked(n_total, 0);
							for (int block = 0; block < blocks; ++block)
							{
								int expect = block * block_rows; // the groups' runs follow each other
								for (int g = 0; g < groups; ++g)
								{
									const fm::StreamRows r = fm::stream_group_rows(block, g, groups, rows, diff, n_total);
									const int run = fm::stream_group_run(g, groups, rows, diff);
									CHECK(r.row0 == expect && run >= 1 && run <= rows, "run %d of group %d starts at %d, expected %d", run, g,
									      r.row0, expect);
									CHECK(r.count >= 0 && r.count <= run, "count %d", r.count);
									expect += run;
									for (int q = 0; q < r.count; ++q)
									{
										CHECK(r.row0 + q < n_total, "%s k %d n %d: row %d", f.name, k, n_total, r.row0 + q);
										if (r.row0 + q < n_total)
										{
											++walked[r.row0 + q];
										}
									}
								}
								CHECK(expect == (block + 1) * block_rows, "a workgroup's runs cover %d rows", expect - block * block_rows);
							}
							for (int r = 0; r < n_total; ++r)
							{
								CHECK(walked[r] == 1, "%s k %d n %d diff %d: row %d walked %d times", f.name, k, n_total, diff, r, walked[r]);
							}
							++cases;
						}
					}
				}
			}
			}
		}
	}
	std::printf("streaming gemv: %ld launch geometries walked\n", cases);
}

// ---- tiled prompt attention -----------------------------------------------------------------------
static void test_attention_tiles()
{
	constexpr int q_tile = 64, key_tile = 64;
	long cases = 0;
	for (int m : { 16, 17, 63, 64, 65, 100, 512, 2048 })
	{
		for (int past : { 0, 1, 5, 63, 64, 1000 })
		{
			const int cache_rows = past + m; // rows the cache is guaranteed to hold
			for (int tile = 0; tile < (m + q_tile - 1) / q_tile; ++tile)
			{
				const int kv_len = fm::attn_tile_kv_len(past, tile * q_tile, q_tile, m);
				CHECK(kv_len >= 1 && kv_len <= cache_rows, "m %d past %d tile %d: kv_len %d", m, past, tile, kv_len);
				// the last row of the tile sees keys 0 .. past + row
				const int last_row = (tile * q_tile + q_tile < m ? tile * q_tile + q_tile : m) - 1;
				CHECK(kv_len == past + last_row + 1, "kv_len %d", kv_len);
				const int n_key_tiles = (kv_len + key_tile - 1) / key_tile;
				std::vector<int> seen(kv_len, 0);
				for (int kt = 0; kt < n_key_tiles + 2; ++kt) // the kernel re-reads the last tile past the end
				{
					const int t = fm::imin(kt, n_key_tiles - 1);
					for (int idx = 0; idx < key_tile; ++idx)
					{
						const int key = fm::attn_tile_key(t, key_tile, idx, kv_len);
						CHECK(key >= 0 && key < kv_len, "m %d past %d: key %d of %d", m, past, key, kv_len);
						if (kt < n_key_tiles && t * key_tile + idx < kv_len)
						{
							++seen[key];
						}
					}
				}
				for (int key = 0; key < kv_len; ++key)
				{
					CHECK(seen[key] == 1, "m %d past %d: key %d staged %d times", m, past, key, seen[key]);
				}
				++cases;
			}
		}
	}
	std::printf("attention tiles: %ld query tiles walked\n", cases);
}

// ---- decoder-block kernel: rows dealt out per team, column segments of the output projection ----
static void test_team_rows_and_segments()
{
	long cases = 0;
	// first phase: every row of every matrix is walked exactly once over the eight teams
	for (int n0 : { 4096, 2048, 1024 })
	{
		for (int n1 : { 4096, 1024, 512, 0 })
		{
			const int n2 = n1;
			std::vector<int> seen0(n0, 0), seen1(n1, 0), seen2(n2, 0);
			const int per_team = (n0 >> 3) + (n1 >> 3) + (n2 >> 3);
			for (int team = 0; team < 8; ++team)
			{
				for (int v = 0; v < per_team; ++v)
				{
					const fm::TeamRow r = fm::team_row(v, team, n0, n1, n2);
					std::vector<int>& seen = r.m == 0 ? seen0 : (r.m == 1 ? seen1 : seen2);
					CHECK(r.m >= 0 && r.m <= 2 && r.local >= 0 && r.local < static_cast<int>(seen.size()),
					      "team %d row %d -> matrix %d row %d", team, v, r.m, r.local);
					if (r.local >= 0 && r.local < static_cast<int>(seen.size()))
					{
						++seen[r.local];
					}
					++cases;
				}
			}
			for (const std::vector<int>* seen : { &seen0, &seen1, &seen2 })
			{
				for (size_t i = 0; i < seen->size(); ++i)
				{
					CHECK((*seen)[i] == 1, "n %d %d: row %zu walked %d times", n0, n1, i, (*seen)[i]);
				}
			}
		}
	}
	// third phase: 4096 x 4096 output projection, team t owns 512 columns (two 256-element chunks) of
	// every row; a wavefront's fetch holds the segments of eight consecutive rows and must look like a
	// 4096-wide slice of a row made of those segments
	for (const Format& f : kFormats)
	{
		const int seg_bytes = 2 * f.chunk_bytes;
		if (seg_bytes % 16 != 0)
		{
			continue; // the launcher sends such a format down the separate launches
		}
		const int n = 4096, row_bytes = 16 * f.chunk_bytes, seg_pieces = seg_bytes / 16, rows_per_fetch = 8;
		CHECK(seg_pieces * rows_per_fetch * 16 == f.stream_slice, "%s: eight segments are not one slice", f.name);
		const int loads = (f.stream_slice + 1023) / 1024;
		const uintptr_t base = 7 * kPage; // page-exact tensor: 4096 rows x 16 chunks
		const uintptr_t end = base + static_cast<size_t>(n) * row_bytes;
		std::vector<unsigned char> covered(static_cast<size_t>(n) * row_bytes, 0);
		for (int block = 0; block < 256; ++block)
		{
			const int team = block & 7, place = block >> 3;
			for (int wave = 0; wave < 8; ++wave)
			{
				for (int fetch = 0; fetch < 2; ++fetch)
				{
					const int row0 = place * 128 + (wave * 2 + fetch) * rows_per_fetch;
					std::map<int, uintptr_t> slot;
					for (int i = 0; i < loads; ++i)
					{
						for (int lane = 0; lane < 64; ++lane)
						{
							const fm::SegmentPiece sp = fm::segment_piece(i, lane, seg_pieces, rows_per_fetch);
							if (!sp.issued)
							{
								continue;
							}
							CHECK(sp.row >= 0 && sp.row < rows_per_fetch && sp.offset + 16 <= static_cast<uint32_t>(seg_bytes),
							      "%s: piece row %d offset %u", f.name, sp.row, sp.offset);
							const uintptr_t from = base + static_cast<size_t>(row0 + sp.row) * row_bytes +
							                       static_cast<size_t>(team) * seg_bytes + sp.offset;
							CHECK(from % 16 == 0 && from >= base && from + 16 <= end, "%s: piece at %#zx outside the tensor", f.name,
							      static_cast<size_t>(from));
							slot[1024 * i + 16 * lane] = from;
							if (from >= base && from + 16 <= end)
							{
								for (int b = 0; b < 16; ++b)
								{
									++covered[from - base + b];
								}
							}
							++cases;
						}
					}
					// the slot, read as a slice: byte b of row r's segment sits at r * seg_bytes + b
					for (int r = 0; r < rows_per_fetch; ++r)
					{
						for (int b = 0; b < seg_bytes; b += 16)
						{
							const auto it = slot.find(r * seg_bytes + b);
							const uintptr_t want = base + static_cast<size_t>(row0 + r) * row_bytes + static_cast<size_t>(team) * seg_bytes + b;
							CHECK(it != slot.end() && it->second == want, "%s: slot byte %d of row %d", f.name, b, r);
						}
					}
				}
			}
		}
		for (size_t i = 0; i < covered.size(); ++i)
		{
			if (covered[i] != 1)
			{
				CHECK(false, "%s: byte %zu of the projection fetched %d times", f.name, i, covered[i]);
				break;
			}
		}
	}
	std::printf("team rows and column segments: %ld rows and pieces walked\n", cases);
}

// The K ranges of the tiled GEMM: whatever the split, the ranges tile [0, chunks) in order; and
// whenever the launcher's condition for several groups per workgroup holds, the groups of every
// workgroup walk equally many chunks (they pass one set of barriers per chunk: an unequal walk would
// leave a group waiting at a barrier the other never reaches).
static void test_gemm_chunk_ranges()
{
	using namespace litenn_hip::fetch;
	long walked = 0;
	for (int chunks = 1; chunks <= 96; ++chunks)
	{
		for (int grid_z = 1; grid_z <= 4; grid_z *= 2)
		{
			for (int groups = 1; groups <= 2; ++groups)
			{
				const int parts = grid_z * groups;
				int expect_begin = 0;
				for (int part = 0; part < parts; ++part)
				{
					const ChunkRange r = gemm_chunk_range(part, parts, chunks);
					CHECK(r.begin == expect_begin && r.end >= r.begin && r.end <= chunks, "chunks %d parts %d part %d: [%d, %d)",
					      chunks, parts, part, r.begin, r.end);
					expect_begin = r.end;
					walked += r.end - r.begin;
				}
				CHECK(expect_begin == chunks, "chunks %d parts %d: ranges end at %d", chunks, parts, expect_begin);
				if (groups > 1 && gemm_ranges_equal(chunks, parts))
				{
					for (int z = 0; z < grid_z; ++z)
					{
						const ChunkRange g0 = gemm_chunk_range(z * groups, parts, chunks);
						const ChunkRange g1 = gemm_chunk_range(z * groups + 1, parts, chunks);
						CHECK(g0.end - g0.begin == g1.end - g1.begin && g0.end > g0.begin,
						      "chunks %d grid z %d: groups of workgroup %d walk %d and %d chunks", chunks, grid_z, z,
						      g0.end - g0.begin, g1.end - g1.begin);
					}
				}
			}
		}
	}
	// an odd chunk count must not pass the launcher's condition
	CHECK(!gemm_ranges_equal(43, 2) && !gemm_ranges_equal(6, 4) && gemm_ranges_equal(16, 4) && !gemm_ranges_equal(1, 2),
	      "the condition for several groups per workgroup");
	std::printf("tiled GEMM K ranges: %ld chunks walked\n", walked);
}

int main()
{
	test_gemm_chunk_ranges();
	test_gemm_weight_pieces();
	test_gemm_stream_pieces();
	test_stream_rows_and_pieces();
	test_attention_tiles();
	test_team_rows_and_segments();
	if (g_failures)
	{
		std::printf("%d checks failed\n", g_failures);
		return 1;
	}
	std::printf("fetch bounds ok\n");
	return 0;
}
