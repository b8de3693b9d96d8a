// Which bytes of a weight tensor, an activation vector or a KV cache a launch may request: the address
// arithmetic of every fetch pattern of the hot kernels, as plain functions that the kernels call on
// the device and that tests/cpp/fetch_bounds_test.cpp calls on the host for every thread of a
// launch.  The test walks page-exact, ragged and minimal shapes and asserts that every requested
// 16-byte piece holds at least one byte of its tensor (an aligned 16-byte piece never crosses a page,
// so such a piece touches mapped memory only) and that the pieces that are consumed cover what the
// kernel needs.  An over-fetch is found there, on the CPU, not by a fault on the GPU.
//
// Nothing here depends on HIP: with a host compiler the functions are ordinary inline functions.
#pragma once

#include <cstddef>
#include <cstdint>

#if defined(__HIPCC__)
#define LITENN_FETCH_FN __host__ __device__ __forceinline__
#else
#define LITENN_FETCH_FN inline
#endif

namespace litenn_hip
{
	namespace fetch
	{
		LITENN_FETCH_FN int imin(int a, int b) { return a < b ? a : b; }
		LITENN_FETCH_FN int imax(int a, int b) { return a > b ? a : b; }

		// ---- matrix-core GEMM: raw weight blocks of one 256-element chunk per row --------------
		// A wavefront owns 16 * ng consecutive rows; their chunks land in its LDS slot row after row
		// as `pieces` 16-byte pieces each.  Formats whose chunks start on 16-byte boundaries take
		// chunk_bytes / 16 pieces; the others (Q2_K 84, Q3_K 110, Q6_K 210 bytes per chunk) start at
		// the 16-byte boundary at or below the chunk and need one piece more for the worst case.
		constexpr int gemm_weight_pieces(int chunk_bytes, bool aligned16)
		{
			return aligned16 ? chunk_bytes / 16 : (chunk_bytes + 14 + 15) / 16;
		}

		struct GemmWeightRequest
		{
			int row;    // 0 .. 16 ng - 1 within the wavefront's rows
			int offset; // byte offset of the piece from the row's first piece: 16 j
			bool issued;
		};

		// load instruction i (0 .. ceil(16 ng pieces / 64) - 1) of `lane`
		LITENN_FETCH_FN GemmWeightRequest gemm_weight_request(int i, int lane, int ng, int pieces)
		{
			const int total = ng * 16 * pieces;
			const int piece = imin(64 * i + lane, total - 1);
			const int row = piece / pieces;
			return { row, 16 * (piece - row * pieces), 64 * (i + 1) <= total || 64 * i + lane < total };
		}

		// rows past the end of the matrix re-read its last row (their products are never stored)
		LITENN_FETCH_FN int gemm_weight_row(int n_base, int row, int n) { return imin(n_base + row, n - 1); }

		// Address of the piece at `offset` of chunk c of the row that starts at `row_start`.  With
		// unaligned chunks `pieces` counts the worst misalignment; with a smaller one the last piece
		// holds no byte of the chunk, and behind the tensor's last chunk it can be the first 16 bytes
		// of a page that is not mapped: such a piece fetches the chunk's first piece again (its slot
		// bytes are never read).
		LITENN_FETCH_FN uintptr_t gemm_weight_piece(uintptr_t row_start, int c, int chunk_bytes, bool aligned16,
		                                            int offset)
		{
			const uintptr_t chunk = row_start + static_cast<size_t>(c) * static_cast<size_t>(chunk_bytes);
			if (aligned16)
			{
				return chunk + static_cast<uintptr_t>(offset);
			}
			const uintptr_t base = chunk & ~uintptr_t{ 15 };
			const uintptr_t from = base + static_cast<uintptr_t>(offset);
			return from >= chunk + static_cast<uintptr_t>(chunk_bytes) ? base : from;
		}

		// where the decoders find the chunk's first byte inside the row's part of the slot
		LITENN_FETCH_FN int gemm_weight_misalignment(uintptr_t row_start, int c, int chunk_bytes, bool aligned16)
		{
			return aligned16
			           ? 0
			           : static_cast<int>((row_start + static_cast<size_t>(c) * static_cast<size_t>(chunk_bytes)) & 15);
		}

		// ---- streaming GEMV: rows HBM -> LDS --------------------------------------------------
		// Wavefront s of a row's `slices` fetches bytes [s * slice_bytes, s * slice_bytes + len) of
		// every row it walks, as loads of 1 KB (64 lanes x 16 bytes).
		LITENN_FETCH_FN uint32_t stream_slice_len(bool whole_slices, uint32_t slice_bytes, uint32_t row_bytes,
		                                          uint32_t slice_off)
		{
			return whole_slices ? slice_bytes : (slice_bytes < row_bytes - slice_off ? slice_bytes : row_bytes - slice_off);
		}

		struct StreamPiece
		{
			uint32_t offset; // from the slice's first byte
			bool issued;
		};

		// Load instruction i of a row, lane `lane`.  Every row takes the same number of instructions
		// whatever the slice's length (the vmcnt bookkeeping is fixed at compile time): an instruction
		// whose 1 KB lies wholly past a short slice still runs in lane 0, which fetches the slice's
		// first 16 bytes again into that (unused) part of the slot.
		LITENN_FETCH_FN StreamPiece stream_row_piece(int i, int lane, uint32_t slice_len, bool whole_slices)
		{
			const uint32_t off = static_cast<uint32_t>(i) * 1024u + static_cast<uint32_t>(lane) * 16u;
			const bool inside = off < slice_len;
			return { inside ? off : 0u, inside || (lane == 0 && !whole_slices) };
		}

		// rows [row0, row0 + count) of the launch that wavefront group g of workgroup `block` walks
		struct StreamRows
		{
			int row0, count;
		};
		// A workgroup's groups walk consecutive runs of its rows.  The first half of the groups walk
		// `run` rows each and the second half `run - diff` (diff > 0 only with an even number of
		// groups): of the two wavefronts that share a SIMD the one that arrived first (the lower
		// index) gets ahead of the other, and the longer run levels the two.
		LITENN_FETCH_FN int stream_group_run(int g, int groups, int run, int diff)
		{
			return 2 * g < groups ? run : run - diff;
		}
		LITENN_FETCH_FN int stream_group_first(int g, int groups, int run, int diff)
		{
			const int half = groups / 2;
			return 2 * g < groups ? g * run : g * run - (g - half) * diff;
		}
		LITENN_FETCH_FN int stream_block_rows(int groups, int run, int diff) { return groups * run - (groups / 2) * diff; }
		LITENN_FETCH_FN StreamRows stream_group_rows(int block, int g, int groups, int run, int diff, int n_total)
		{
			const int row0 = block * stream_block_rows(groups, run, diff) + stream_group_first(g, groups, run, diff);
			return { row0, imax(0, imin(stream_group_run(g, groups, run, diff), n_total - row0)) };
		}

		// first float of the 128-bit activation load j of thread `tid` (clamped: every lane issues
		// every load)
		LITENN_FETCH_FN int stream_x_index(int tid, int j, int threads, int k) { return imin((tid + j * threads) * 4, k - 4); }

		// ---- decoder-block kernel: rows dealt out per XCD, and the output projection's columns ---
		// The launch's 256 workgroups form eight teams of 32 (workgroup b: team b % 8, place b / 8;
		// the dispatcher deals workgroups to the card's eight XCDs in that order, so a team shares
		// an L2).  Team t takes an eighth of the rows of each of the up to three matrices of the
		// first phase: virtual row v of the team lies in matrix m at row t * (n[m] / 8) + r.
		struct TeamRow
		{
			int m, local;
		};
		LITENN_FETCH_FN TeamRow team_row(int v, int team, int n0, int n1, int n2)
		{
			const int r0 = n0 >> 3, r1 = n1 >> 3, r2 = n2 >> 3;
			if (v < r0)
			{
				return { 0, team * r0 + v };
			}
			if (v < r0 + r1)
			{
				return { 1, team * r1 + (v - r0) };
			}
			return { 2, team * r2 + imin(v - r0 - r1, r2 > 0 ? r2 - 1 : 0) };
		}

		// The third phase multiplies a column slice of the output projection: team t owns `seg_bytes`
		// bytes of every row (the blocks of its heads' columns), from byte t * seg_bytes of the row.
		// A wavefront fetches the segments of `rows_per_fetch` consecutive rows (4096 weights in all)
		// as one run of 16-byte pieces, piece p of the run being piece p % seg_pieces of row
		// p / seg_pieces; load instruction i moves pieces 64 i .. 64 i + 63 to consecutive LDS
		// addresses, so the slot holds what a 4096-wide slice of a row would.
		struct SegmentPiece
		{
			int row;         // 0 .. rows_per_fetch - 1
			uint32_t offset; // from the segment's first byte
			bool issued;
		};
		LITENN_FETCH_FN SegmentPiece segment_piece(int i, int lane, int seg_pieces, int rows_per_fetch)
		{
			const int total = seg_pieces * rows_per_fetch;
			const int p = 64 * i + lane;
			const int q = imin(p, total - 1);
			return { q / seg_pieces, static_cast<uint32_t>(q % seg_pieces) * 16u, p < total };
		}

		// ---- tiled GEMM: the chunks of K a group of wavefronts walks ------------------------------
		// K (in 256-element chunks) is cut into `parts` consecutive ranges: grid z x the K groups of a
		// workgroup, part = blockIdx.z * groups + group
		struct ChunkRange
		{
			int begin, end;
		};
		LITENN_FETCH_FN ChunkRange gemm_chunk_range(int part, int parts, int chunks)
		{
			return { part * chunks / parts, (part + 1) * chunks / parts };
		}
		// The K groups of one workgroup pass the same barriers, one set per chunk: a launch with more than
		// one group per workgroup is only made when this holds (every range is then equally long)
		LITENN_FETCH_FN bool gemm_ranges_equal(int chunks, int parts)
		{
			return parts > 0 && chunks >= parts && chunks % parts == 0;
		}

		// ---- tiled prompt attention: key / value rows of a 64-key tile -------------------------
		// keys any query row of the 64-row tile starting at q_first may see
		LITENN_FETCH_FN int attn_tile_kv_len(int past, int q_first, int q_tile, int m)
		{
			return past + imin(m, q_first + q_tile) - 1 + 1;
		}
		// cache row fetched for slot `idx` (0 .. 63) of key tile kt: past the end the last key is re-read
		LITENN_FETCH_FN int attn_tile_key(int kt, int key_tile, int idx, int kv_len)
		{
			return imin(kt * key_tile + idx, kv_len - 1);
		}
	} // namespace fetch
} // namespace litenn_hip
