// Plan files of the SDDMM engine: a plan's device arrays and launch descriptors under a header with
// the key it was built for.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstring>
#include <new>
#include <unistd.h>
#include "plan.hpp"
#include "build_id.h"

using namespace sddmm;

// ---- plan files -------------------------------------------------------------
// A plan file is the plan's device arrays and launch descriptors under a header with the key it
// was built for.  Device pointers are stored as (allocation number + 1) << 44 | byte offset.
namespace {

struct PlanFileHeader {
    char magic[8];
    uint32_t version, sizeof_launch, sizeof_info, sizeof_options;
    int64_t n_rows, n_cols, nnz;
    int32_t K, requested_kernel;
    uint64_t pattern_hash;
    uint64_t n_allocs, n_launches;
    uint64_t code_row_ptr, code_col, code_val;
    char build[40];          // SDDMM_BUILD_ID of the library that wrote the file: a hash of its sources
    uint64_t meta_checksum;  // over info, options, allocation sizes and launch table as they lie in the file
    uint64_t data_checksum;  // over the arrays, in pieces of kPlanPiece bytes per allocation (see piece_hash)
};
constexpr char kPlanMagic[8] = {'S', 'D', 'D', 'M', 'M', 'P', 'L', 'N'};
constexpr uint32_t kPlanVersion = 4;
constexpr size_t kPlanPiece = (size_t)16 << 20;  // arrays are read, copied and check-summed in pieces of this size

// Hash of one piece of an array: four interleaved multiply-add chains over its 8-byte words (so that a
// thread runs at memory speed), folded with the piece's place in the file.  The file's checksum is the
// wrapping sum of its pieces' hashes, whatever order they are read in.
uint64_t piece_hash(const void *data, size_t n, uint64_t alloc, uint64_t piece)
{
    const unsigned char *b = (const unsigned char *)data;
    uint64_t h[4] = {0x243f6a8885a308d3ull, 0x13198a2e03707344ull, 0xa4093822299f31d0ull, 0x082efa98ec4e6c89ull};
    constexpr uint64_t kMul = 0x9e3779b97f4a7c15ull;
    size_t i = 0;
    for (; i + 32 <= n; i += 32) {
        uint64_t w[4];
        memcpy(w, b + i, 32);
        for (int k = 0; k < 4; ++k) h[k] = (h[k] ^ w[k]) * kMul + (h[k] >> 29);
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    memcpy(tail, b + i, n - i);
    for (int k = 0; k < 4; ++k) h[k] = (h[k] ^ tail[k]) * kMul + (h[k] >> 29);
    uint64_t x = (uint64_t)n;
    for (int k = 0; k < 4; ++k) x = mix64(x ^ h[k]);
    return mix64(x ^ (alloc << 32) ^ piece);
}

// a launch descriptor read from a file must describe a launch this library could have planned
bool launch_plausible(const Launch &L, int64_t nnz)
{
    const int64_t slack = 2 * nnz + (1 << 20);  // padded streams stay well below twice the nonzeros + per-item rounding
    return L.fn_kind >= 1 && L.fn_kind <= 5 && L.grid > 0 && L.grid <= (1 << 24) && L.block >= 64 && L.block <= 1024 &&
           L.block % 64 == 0 && L.lds >= 0 && L.lds <= kLdsMaxBytes && L.nnz >= 0 && L.nnz <= nnz && L.rows >= 0 &&
           L.positions >= 0 && L.positions <= slack + 62 * nnz && L.k_slice >= 0 && L.fn_nwm >= 0 && L.fn_nwm <= 8 &&
           L.ta.n_items >= 0 && L.ta.n_units >= 0 && L.ka.n_items >= 0 && L.ta.mf_groups >= 0 && L.ta.mf_n_cb >= 0;
}
constexpr uint64_t kScratchBit = 1ull << 63;
constexpr uint64_t kBorrowedRowPtr = (1ull << 63) | 1, kBorrowedCol = (1ull << 63) | 2;

// every pointer of a launch that refers to memory the plan owns
void launch_pointer_fields(Launch &L, std::vector<void *> &fields)
{
    fields = {&L.ka.perm, &L.ka.scol, &L.ka.seg_row, &L.ka.batch_seg, &L.ka.batch_mask, &L.ka.items,
            &L.ta.perm, &L.ta.scol, &L.ta.grow, &L.ta.scol16, &L.ta.pbase, &L.ta.btype, &L.ta.part, &L.ta.sink, &L.ta.unit_ptr,
            &L.ta.unit_tile, &L.ta.items, &L.ta.mf_hp, &L.ta.mf_wp, &L.ta.mf_rowinfo, &L.ta.mf_rows,
            &L.sa.items, &L.sa.b_off, &L.sa.b_p0, &L.sa.b_len, &L.sa.cols, &L.sa.part, &L.sa.row_part_ptr, &L.sa.part_slot,
            &L.sa.sum_rows, &L.sa.gather_rows,
            &L.pa.slot_row, &L.pa.panel_tiles,
            &L.da.slot_rows, &L.da.slot_cols, &L.da.slot_range, &L.da.nz_p, &L.da.nz_rc,
            &L.sval, &L.perm};
}

bool encode_pointer(const sddmm_plan *P, const void *p, uint64_t *code)
{
    *code = 0;
    if (!p) return true;
    for (size_t i = 0; i < P->owned.size(); ++i) {
        const char *b = (const char *)P->owned[i].p;
        if ((const char *)p >= b && (const char *)p < b + P->owned[i].bytes) {
            *code = ((uint64_t)(i + 1) << 44) | (uint64_t)((const char *)p - b);
            return true;
        }
    }
    return false;
}

bool decode_pointer(const sddmm_plan *P, uint64_t code, void **p)
{
    *p = nullptr;
    if (!code) return true;
    const uint64_t i = (code >> 44), off = code & ((1ull << 44) - 1);
    if (i < 1 || i > P->owned.size() || off >= P->owned[i - 1].bytes) return false;
    *p = (char *)P->owned[i - 1].p + off;
    return true;
}

bool same_options(const sddmm_plan_options &a, const sddmm_plan_options &b)
{
    // field by field (the structure may hold padding); how the values got there (ignore_env) is not part of the key
    const int la = a.tile_lanes < 0 ? 0 : a.tile_lanes, lb = b.tile_lanes < 0 ? 0 : b.tile_lanes;
    return a.kernel == b.kernel && a.tile_size_x == b.tile_size_x && a.tile_size_y == b.tile_size_y && a.k_slice == b.k_slice &&
           la == lb && a.tile_waves == b.tile_waves && a.tile_assign == b.tile_assign && a.tile_few_blocks == b.tile_few_blocks &&
           a.tile_short_batches == b.tile_short_batches && a.tile_deal == b.tile_deal && a.tile_runs == b.tile_runs && a.fuse_slices == b.fuse_slices &&
           a.gather_lanes == b.gather_lanes && a.gather_padded == b.gather_padded && a.gather_sink == b.gather_sink &&
           a.row_padded == b.row_padded && a.unpadded_tile == b.unpadded_tile && a.dense_blocks == b.dense_blocks &&
           a.dense_permille == b.dense_permille && a.dense_rb_group == b.dense_rb_group &&
           a.matrix_rows == b.matrix_rows && a.matrix_permille == b.matrix_permille && a.matrix_waves == b.matrix_waves &&
           a.spmm_stream == b.spmm_stream &&
           a.gather_slab_cols == b.gather_slab_cols && a.gather_panel_rows == b.gather_panel_rows &&
           a.dense_min_nnz == b.dense_min_nnz && a.panel_bytes == b.panel_bytes && a.short_row_max == b.short_row_max &&
           a.stage_factor == b.stage_factor && a.split_min_nnz == b.split_min_nnz;
}

struct FileCloser { FILE *f; ~FileCloser() { if (f) fclose(f); } };

int load_plan_file(const char *path, int64_t n_rows, int64_t n_cols, int64_t nnz, int32_t K, const sddmm_plan_options *opt_in,
                   const uint64_t *want_hash, const int32_t *d_row_ptr, const int32_t *d_col_ind, sddmm_plan **out)
{
    auto t0 = std::chrono::steady_clock::now();
    if (int rc = device_ok()) return rc;
    FILE *f = fopen(path, "rb");
    if (!f) return fail(SDDMM_ERR_IO, "sddmm_plan_load: cannot open %s", path);
    FileCloser fc{f};
    PlanFileHeader h;
    if (fread(&h, sizeof h, 1, f) != 1 || memcmp(h.magic, kPlanMagic, 8) != 0)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is not a plan file", path);
    h.build[sizeof h.build - 1] = 0;
    if (h.version != kPlanVersion || h.sizeof_launch != sizeof(Launch) || h.sizeof_info != sizeof(sddmm_plan_info) ||
        h.sizeof_options != sizeof(sddmm_plan_options) || strncmp(h.build, SDDMM_BUILD_ID, sizeof h.build - 1) != 0)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was written by another build of the library (%s, this one is %s)", path,
                    h.build, SDDMM_BUILD_ID);
    if (h.n_rows != n_rows || h.n_cols != n_cols || h.nnz != nnz || h.K != K)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s holds a plan for %lld x %lld, nnz %lld, K %d, not for %lld x %lld, nnz %lld, K %d",
                    path, (long long)h.n_rows, (long long)h.n_cols, (long long)h.nnz, h.K, (long long)n_rows, (long long)n_cols,
                    (long long)nnz, K);
    if (want_hash && *want_hash != h.pattern_hash)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was built for another sparsity pattern", path);
    if (h.n_allocs > (1u << 20) || h.n_launches > (1u << 16)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged", path);
    sddmm_plan *P = new (std::nothrow) sddmm_plan;
    if (!P) return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load: out of memory");
    struct Guard { sddmm_plan *p; ~Guard() { delete p; } } guard{P};
    if (fread(&P->info, sizeof P->info, 1, f) != 1 || fread(&P->options, sizeof P->options, 1, f) != 1)
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    if (opt_in) {
        sddmm_plan_options want = *opt_in;
        apply_env_overrides(want);
        if (!same_options(want, P->options))
            return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s was built with other plan options", path);
    }
    std::vector<uint64_t> sizes((size_t)h.n_allocs);
    if (h.n_allocs && fread(sizes.data(), 8, sizes.size(), f) != sizes.size())
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    P->launches.resize((size_t)h.n_launches);
    if (h.n_launches && fread((void *)P->launches.data(), sizeof(Launch), P->launches.size(), f) != P->launches.size())
        return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
    {
        uint64_t m = piece_hash(&P->info, sizeof P->info, 0, 0) + piece_hash(&P->options, sizeof P->options, 0, 1) +
                     piece_hash(sizes.data(), sizes.size() * 8, 0, 2) +
                     piece_hash((const void *)P->launches.data(), P->launches.size() * sizeof(Launch), 0, 3);
        if (m != h.meta_checksum) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (launch table checksum)", path);
        for (const Launch &L : P->launches)
            if (!launch_plausible(L, nnz)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (launch descriptor)", path);
    }
    // The arrays: pieces of 16 MiB are read (pread) by a few threads, each into its own pair of pinned
    // staging buffers, check-summed there and copied to the device on the thread's own stream as they arrive.
    constexpr size_t kPiece = kPlanPiece;
    const long data_at = ftell(f);
    if (data_at < 0) return fail(SDDMM_ERR_IO, "sddmm_plan_load: cannot seek in %s", path);
    struct Piece { void *dst; uint64_t file_off; size_t n; uint64_t alloc, piece; };
    std::vector<Piece> pieces;
    int64_t total = 0;
    {
        uint64_t at = (uint64_t)data_at, alloc = 0;
        for (uint64_t word : sizes) {
            ++alloc;
            const bool scratch = (word & kScratchBit) != 0;
            const uint64_t bytes = word & ~kScratchBit;
            if (bytes == 0 || bytes > ((uint64_t)1 << 40)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged", path);
            void *d = nullptr;
            HIP_TRY(hipMalloc(&d, bytes));
            P->owned.push_back({d, (size_t)bytes, scratch});
            total += (int64_t)bytes;
            if (scratch) continue;
            for (uint64_t off = 0; off < bytes; off += kPiece)
                pieces.push_back({(char *)d + off, at + off, (size_t)std::min<uint64_t>(kPiece, bytes - off), alloc, off / kPiece});
            at += bytes;
        }
    }
    const int n_readers = (int)std::max<size_t>(1, std::min<size_t>({(size_t)8, (size_t)hw_threads(), pieces.size()}));
    std::vector<int> reader_rc((size_t)n_readers, 0);  // 0 ok, 1 short read, 2 HIP error
    std::vector<uint64_t> reader_sum((size_t)n_readers, 0);
    const int fd = fileno(f);
    {
        std::vector<std::thread> th;
        auto reader = [&](int t) {
                void *stage[2] = {nullptr, nullptr};
                hipEvent_t done[2] = {nullptr, nullptr};
                hipStream_t st = nullptr;
                bool ok = hipStreamCreate(&st) == hipSuccess;
                for (int i = 0; i < 2 && ok; ++i)
                    ok = hipHostMalloc(&stage[i], kPiece, hipHostMallocDefault) == hipSuccess && hipEventCreate(&done[i]) == hipSuccess;
                int turn = 0;
                for (size_t k = (size_t)t; ok && k < pieces.size(); k += (size_t)n_readers, turn ^= 1) {
                    const Piece &pc = pieces[k];
                    if (hipEventSynchronize(done[turn]) != hipSuccess) { ok = false; break; }  // (never recorded: complete)
                    size_t got = 0;
                    while (got < pc.n) {
                        const ssize_t r = pread(fd, (char *)stage[turn] + got, pc.n - got, (off_t)(pc.file_off + got));
                        if (r <= 0) break;
                        got += (size_t)r;
                    }
                    if (got != pc.n) { reader_rc[(size_t)t] = 1; break; }
                    reader_sum[(size_t)t] += piece_hash(stage[turn], pc.n, pc.alloc, pc.piece);
                    ok = hipMemcpyAsync(pc.dst, stage[turn], pc.n, hipMemcpyHostToDevice, st) == hipSuccess &&
                         hipEventRecord(done[turn], st) == hipSuccess;
                }
                if (st) ok = (hipStreamSynchronize(st) == hipSuccess) && ok;
                if (!ok && !reader_rc[(size_t)t]) reader_rc[(size_t)t] = 2;
                for (int i = 0; i < 2; ++i) { if (stage[i]) (void)hipHostFree(stage[i]); if (done[i]) (void)hipEventDestroy(done[i]); }
                if (st) (void)hipStreamDestroy(st);
        };
        // (a thread that cannot be started: its share is read by this one)
        for (int t = 0; t < n_readers; ++t) {
            try {
                th.emplace_back(reader, t);
            } catch (const std::system_error &) {
                reader(t);
            }
        }
        for (auto &x : th) x.join();
    }
    for (int rc : reader_rc) {
        if (rc == 1) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is cut short", path);
        if (rc == 2) return fail(SDDMM_ERR_HIP, "sddmm_plan_load: copying %s to the device failed", path);
    }
    HIP_TRY(hipDeviceSynchronize());
    {
        uint64_t sum = 0;
        for (uint64_t x : reader_sum) sum += x;
        if (sum != h.data_checksum) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (array checksum)", path);
    }
    // pointers
    void *q = nullptr;
    std::vector<void *> fields;
    for (Launch &L : P->launches) {
        launch_pointer_fields(L, fields);
        for (void *field : fields) {
            uint64_t code;
            memcpy(&code, field, 8);
            if (!decode_pointer(P, code, &q)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (bad reference)", path);
            memcpy(field, &q, 8);
        }
        L.ka.col_ind = nullptr; L.ka.val = nullptr; L.ka.W = L.ka.H = nullptr; L.ka.out = nullptr; L.ka.sval = nullptr;
        L.ka.row_ptr = nullptr; L.ka.batch_row = nullptr;
        L.ta.sval = nullptr; L.ta.val = nullptr; L.ta.W = L.ta.H = nullptr; L.ta.out = nullptr;
        L.pa.row_ptr = nullptr; L.pa.col_ind = nullptr; L.pa.val = nullptr; L.pa.W = L.pa.H = nullptr; L.pa.out = nullptr;
        L.da.nz_val = nullptr; L.da.val = nullptr; L.da.W = L.da.H = nullptr; L.da.out = nullptr;
        if (int rc = resolve_functions(L)) return rc;
    }
    auto place = [&](uint64_t code, const int32_t *borrowed, uint64_t marker, const void **dst) -> bool {
        if (code == marker) { *dst = borrowed; return borrowed != nullptr; }
        void *x = nullptr;
        if (!decode_pointer(P, code, &x)) return false;
        *dst = x;
        return true;
    };
    const void *rp = nullptr, *ci = nullptr;
    if (!place(h.code_row_ptr, d_row_ptr, kBorrowedRowPtr, &rp) || !place(h.code_col, d_col_ind, kBorrowedCol, &ci))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_load: %s holds a plan over a device-resident pattern: pass d_row_ptr and d_col_ind "
                                   "(sddmm_plan_load_device)", path);
    P->d_row_ptr = (const int32_t *)rp; P->d_col = (const int32_t *)ci;
    if (!decode_pointer(P, h.code_val, &q)) return fail(SDDMM_ERR_FORMAT, "sddmm_plan_load: %s is damaged (bad reference)", path);
    P->d_val = (float *)q;
    P->requested_kernel = h.requested_kernel;
    P->pattern_hash = h.pattern_hash;
    P->info.device_bytes = total;
    assign_workspace(P);
    P->info.plan_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    guard.p = nullptr;
    *out = P;
    return SDDMM_OK;
}

}  // namespace

int sddmm_plan_save(const sddmm_plan *plan, const char *path)
{
    if (!plan || !path) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: NULL argument");
    try {
        PlanFileHeader h;
        memset(&h, 0, sizeof h);
        memcpy(h.magic, kPlanMagic, 8);
        h.version = kPlanVersion; h.sizeof_launch = sizeof(Launch); h.sizeof_info = sizeof(sddmm_plan_info);
        h.sizeof_options = sizeof(sddmm_plan_options);
        h.n_rows = plan->info.n_rows; h.n_cols = plan->info.n_cols; h.nnz = plan->info.nnz; h.K = plan->info.K;
        h.requested_kernel = plan->requested_kernel; h.pattern_hash = plan->pattern_hash;
        h.n_allocs = plan->owned.size(); h.n_launches = plan->launches.size();
        strncpy(h.build, SDDMM_BUILD_ID, sizeof h.build - 1);
        if (!encode_pointer(plan, plan->d_row_ptr, &h.code_row_ptr)) h.code_row_ptr = kBorrowedRowPtr;
        if (!encode_pointer(plan, plan->d_col, &h.code_col)) h.code_col = kBorrowedCol;
        if (!encode_pointer(plan, plan->d_val, &h.code_val)) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: values outside the plan's memory");
        std::vector<Launch> ls(plan->launches);
        std::vector<void *> fields;
        for (Launch &L : ls) {
            launch_pointer_fields(L, fields);
            for (void *field : fields) {
                const void *p;
                memcpy(&p, field, 8);
                uint64_t code;
                if (!encode_pointer(plan, p, &code)) return fail(SDDMM_ERR_ARG, "sddmm_plan_save: a launch refers to memory outside the plan");
                memcpy(field, &code, 8);
            }
            L.fn = nullptr; L.pfn = nullptr; L.tfn = nullptr; L.dfn = nullptr;
            for (auto &row : L.tfns) for (auto &fp : row) fp = nullptr;
        }
        HIP_TRY(hipDeviceSynchronize());  // a set_values still in flight has to land first
        // written under a temporary name and renamed when complete: an interrupted save leaves no file under `path`
        const std::string tmp = std::string(path) + ".tmp";
        FILE *f = fopen(tmp.c_str(), "wb");
        if (!f) return fail(SDDMM_ERR_IO, "sddmm_plan_save: cannot create %s", tmp.c_str());
        struct Unlink { const std::string &p; bool armed = true; ~Unlink() { if (armed) (void)remove(p.c_str()); } } cleanup{tmp};
        bool ok;
        {
            FileCloser fc{f};
            std::vector<uint64_t> sizes;  // (bit 63: scratch, no contents in the file)
            for (const auto &o : plan->owned) sizes.push_back((uint64_t)o.bytes | (o.scratch ? kScratchBit : 0));
            h.meta_checksum = piece_hash(&plan->info, sizeof plan->info, 0, 0) + piece_hash(&plan->options, sizeof plan->options, 0, 1) +
                              piece_hash(sizes.data(), sizes.size() * 8, 0, 2) +
                              piece_hash((const void *)ls.data(), ls.size() * sizeof(Launch), 0, 3);
            ok = fwrite(&h, sizeof h, 1, f) == 1 && fwrite(&plan->info, sizeof plan->info, 1, f) == 1 &&
                 fwrite(&plan->options, sizeof plan->options, 1, f) == 1;
            ok = ok && (sizes.empty() || fwrite(sizes.data(), 8, sizes.size(), f) == sizes.size());
            ok = ok && (ls.empty() || fwrite((const void *)ls.data(), sizeof(Launch), ls.size(), f) == ls.size());
            std::vector<char> buf;
            uint64_t alloc = 0;
            for (const auto &o : plan->owned) {
                ++alloc;
                if (o.scratch) continue;
                for (size_t off = 0; ok && off < o.bytes; off += kPlanPiece) {
                    const size_t n = std::min(kPlanPiece, o.bytes - off);
                    buf.resize(n);
                    HIP_TRY(hipMemcpy(buf.data(), (const char *)o.p + off, n, hipMemcpyDeviceToHost));
                    h.data_checksum += piece_hash(buf.data(), n, alloc, off / kPlanPiece);
                    ok = fwrite(buf.data(), 1, n, f) == n;
                }
            }
            // the header once more, now with the checksum of what followed it
            ok = ok && fseek(f, 0, SEEK_SET) == 0 && fwrite(&h, sizeof h, 1, f) == 1 && fflush(f) == 0;
        }
        if (!ok) return fail(SDDMM_ERR_IO, "sddmm_plan_save: write to %s failed", tmp.c_str());
        if (rename(tmp.c_str(), path) != 0) return fail(SDDMM_ERR_IO, "sddmm_plan_save: cannot rename %s to %s", tmp.c_str(), path);
        cleanup.armed = false;
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_save: %s", e.what());
    }
    return SDDMM_OK;
}

int sddmm_plan_load(const char *path, const sddmm_coo *S, int32_t K, const sddmm_plan_options *opt, sddmm_plan **out)
{
    if (!path || !S || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_load: NULL argument");
    *out = nullptr;
    if (S->sorted != 1) return fail(SDDMM_ERR_UNSORTED, "sddmm_plan_load: matrix is not (row, col)-sorted");
    try {
        std::vector<int32_t> rp;
        build_row_ptr(*S, rp);
        const uint64_t hash = pattern_hash_host(S->n_rows, S->nnz, rp.data(), S->cols.data());
        return load_plan_file(path, S->n_rows, S->n_cols, S->nnz, K, opt, &hash, nullptr, nullptr, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load: %s", e.what());
    }
}

int sddmm_plan_load_device(const char *path, int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *d_row_ptr,
                           const int32_t *d_col_ind, int32_t K, const sddmm_plan_options *opt, sddmm_plan **out)
{
    if (!path || !out) return fail(SDDMM_ERR_ARG, "sddmm_plan_load_device: NULL argument");
    *out = nullptr;
    if (n_rows < 0 || n_cols < 0 || nnz < 0 || !d_row_ptr || (nnz > 0 && !d_col_ind))
        return fail(SDDMM_ERR_ARG, "sddmm_plan_load_device: bad sizes or NULL arrays");
    if (int rc = device_ok()) return rc;
    try {
        uint64_t hash = 0;
        if (int rc = pattern_hash_device(n_rows, nnz, d_row_ptr, d_col_ind, &hash)) return rc;
        return load_plan_file(path, n_rows, n_cols, nnz, K, opt, &hash, d_row_ptr, d_col_ind, out);
    } catch (const std::exception &e) {
        return fail(SDDMM_ERR_NOMEM, "sddmm_plan_load_device: %s", e.what());
    }
}
