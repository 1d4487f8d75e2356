// Host-side check of the index arithmetic behind the direct global -> LDS tile copies of the kernels (TileDma in
// csrc/mlstm_device.h): compiled for the host only and run on the CPU, it calls the very functions the kernels use.
// For every tile shape, element size and wave count in use, for dense rows and for rows that lie far apart in memory:
//   - the per-lane offsets the kernels keep (blocks it < PERIOD) plus the scalar group step reproduce the direct formula
//     for every block;
//   - every 16-byte piece of the tile (row, chunk) is fetched exactly once, and lands on a distinct 16-byte slot of the
//     LDS tile inside [0, ROWS * D * sizeof(T));
//   - no fetch ends beyond the last byte of the tile's last row: for the last tile of the last head that is the end of the
//     caller's tensor.
// And for the early touch of a row's cache lines in the eight-wave row kernel: no touched word lies beyond the half row.
#include <cstdio>
#include <vector>
#include "mlstm_device.h"

using namespace mlstm;

static int failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { failures++; if (failures < 20) { std::printf(__VA_ARGS__); std::printf("\n"); } } } while (0)

template <typename T, int D, int ROWS, int NT>
static void check_tile(const char* what) {
    using TD = TileDma<T, D, ROWS, NT>;
    using Z = Swz<T, D>;
    const unsigned dense = (unsigned)(D * sizeof(T));
    for (unsigned row_bytes : {dense, dense * 3u * 8u, dense * 97u}) {   // dense rows; a fused [B,S,3,NH,D] projection; far apart
        const long long tile_end = (long long)(ROWS - 1) * row_bytes + dense;   // one past the last byte of the last row
        std::vector<int> seen((size_t)ROWS * Z::CPR, 0), slot((size_t)ROWS * Z::CPR, 0);
        for (int wave = 0; wave < TD::NW; wave++)
            for (int it = 0; it < TD::PER_WAVE; it++)
                for (int lane = 0; lane < 64; lane++) {
                    const unsigned direct = TD::lane_source(it, wave, lane, row_bytes);
                    const unsigned kept = TD::lane_source(it % TD::PERIOD, wave, lane, row_bytes) + (unsigned)(it / TD::PERIOD) * TD::group_bytes(row_bytes);
                    CHECK(direct == kept, "%s D=%d rows=%d: block %d wave %d lane %d: kept offset %u != %u", what, D, ROWS, it, wave, lane, kept, direct);
                    CHECK((long long)direct + 16 <= tile_end, "%s D=%d rows=%d row_bytes=%u: fetch at %u ends beyond the tile (%lld)", what, D, ROWS, row_bytes, direct, tile_end);
                    const unsigned r = direct / row_bytes, c = (direct % row_bytes) / 16;
                    CHECK(r < (unsigned)ROWS && c < (unsigned)Z::CPR && direct % 16 == 0, "%s: fetch at %u is not a piece of the tile", what, direct);
                    if (r < (unsigned)ROWS && c < (unsigned)Z::CPR) seen[(size_t)r * Z::CPR + c]++;
                    // where it lands: block (it * NW + wave), 16 bytes per lane; the reader finds chunk c of row r at c ^ key(r)
                    const unsigned lds = (unsigned)((it * TD::NW + wave) * 1024 + 16 * lane);
                    CHECK(lds + 16 <= (unsigned)(ROWS * D * sizeof(T)), "%s: LDS destination %u outside the tile", what, lds);
                    CHECK(lds == (unsigned)Z::off((int)r, (int)c * Z::EPC), "%s D=%d: piece (%u, %u) lands at %u, readers expect %d", what, D, r, c, lds,
                          Z::off((int)r, (int)c * Z::EPC));
                    slot[lds / 16]++;
                }
        for (size_t k = 0; k < seen.size(); k++) {
            CHECK(seen[k] == 1, "%s D=%d rows=%d: piece %zu fetched %d times", what, D, ROWS, k, seen[k]);
            CHECK(slot[k] == 1, "%s D=%d rows=%d: LDS slot %zu written %d times", what, D, ROWS, k, slot[k]);
        }
    }
}

template <int HALF_ROW_BYTES>
static void check_pieces() {
    // the two lanes of a row load every 16-byte piece of the half row exactly once and stay inside it
    constexpr int NP = row8_pieces_per_lane(HALF_ROW_BYTES);
    std::vector<int> seen(HALF_ROW_BYTES / 16, 0);
    for (int h = 0; h < 2; h++)
        for (int i = 0; i < NP; i++) {
            const int o = row8_piece_offset(i, h, HALF_ROW_BYTES);
            CHECK(o % 16 == 0 && o + 16 <= HALF_ROW_BYTES, "piece %d of lane half %d ends at %d of %d bytes", i, h, o + 16, HALF_ROW_BYTES);
            seen[o / 16]++;
        }
    for (size_t k = 0; k < seen.size(); k++) CHECK(seen[k] == 1, "half row of %d bytes: piece %zu loaded %d times", HALF_ROW_BYTES, k, seen[k]);
}

int main() {
    // 64-row tiles of the row and column kernels (four waves copy; the eight-wave kernel copies with the four waves of a role)
    check_tile<__bf16, 128, 64, 256>("64-row tile, 16-bit");
    check_tile<__bf16, 256, 64, 256>("64-row tile, 16-bit");
    check_tile<__bf16, 64, 64, 256>("64-row tile, 16-bit");
    check_tile<float, 64, 64, 256>("64-row tile, fp32");
    check_tile<float, 128, 64, 256>("64-row tile, fp32");
    // 32-row query tiles and state pieces, 128-row V tiles of cold_kernel
    check_tile<__bf16, 128, 32, 256>("32-row tile");
    check_tile<__bf16, 256, 32, 256>("32-row tile");
    check_tile<__bf16, 128, 128, 256>("128-row tile");
    check_tile<__bf16, 256, 128, 256>("128-row tile");
    // half rows of the dQ pass: the pieces its row sums load, D = 128 and 256, 16-bit
    check_pieces<128>();
    check_pieces<256>();
    if (failures) { std::printf("tile_bounds: %d check(s) failed\n", failures); return 1; }
    std::printf("tile_bounds: ok\n");
    return 0;
}
