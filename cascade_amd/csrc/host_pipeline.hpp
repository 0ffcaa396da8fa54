// Partitions that arrive in host memory and leave to host memory: upload, sort and download run as a three-stage
// pipeline on four streams (one up, one for the sort, two down), so that the transfers of one partition hide behind the sort of another, as the three
// dispatcher threads of the reference overlap them (src/GPU_SACA.cu:1539-1589). Host code only; included by
// cascade_hip.hip after the C ABI's definitions.
#pragma once

#include <condition_variable>
#include <thread>

// pieces a download is cut into, each on a stream of its own (12 texts of 2^26 symbols, pinned memory, whole job:
// 152 ms with one piece, where one copy engine brings 29 GB/s down; 106 ms with two, 46 GB/s; 120 ms with four).
// The uploads (2 of the 7 bytes per suffix) travel on one stream: with the sort's stream that makes four streams, one
// per hardware queue a process has by default; a fifth would share a queue with another and wait behind it.
#ifndef CSA_PIPELINE_COPY_WAYS
#define CSA_PIPELINE_COPY_WAYS 2
#endif

namespace {

// Progress of the three stages over the list of partitions: stage s has finished partitions [0, done[s]).
struct HostPipeline {
    std::mutex mu;
    std::condition_variable cv;
    u32 uploaded = 0, sorted = 0, downloaded = 0;
    int status = CSA_OK;
    char message[512] = "";

    // Blocks until `counter` reaches `target` or a stage has failed; false after a failure.
    bool wait_for(const u32& counter, u32 target)
    {
        std::unique_lock<std::mutex> lock(mu);
        cv.wait(lock, [&] { return counter >= target || status != CSA_OK; });
        return status == CSA_OK;
    }
    void advance(u32& counter)
    {
        {
            std::lock_guard<std::mutex> lock(mu);
            ++counter;
        }
        cv.notify_all();
    }
    void failed(int code)
    {
        {
            std::lock_guard<std::mutex> lock(mu);
            if (status == CSA_OK) {
                status = code;
                snprintf(message, sizeof(message), "%s", g_err); // the failing thread's message, for the caller's thread
            }
        }
        cv.notify_all();
    }
};

// One transfer, cut into `ways` pieces that travel on as many streams at once (one copy engine moves a piece; the link
// has room for more than one engine's rate); returns when all of it is there.
int copy_through(hipStream_t* streams, u32 ways, void* dst, const void* src, u64 bytes, hipMemcpyKind kind)
{
    if (bytes == 0)
        return CSA_OK;
    if (bytes < (1u << 22))
        ways = 1;
    const u64 piece = ((bytes + ways - 1) / ways + 4095) & ~(u64)4095;
    for (u32 w = 0; w < ways; ++w) {
        const u64 at = (u64)w * piece;
        if (at >= bytes)
            break;
        const u64 len = bytes - at < piece ? bytes - at : piece;
        HIP_TRY(hipMemcpyAsync(static_cast<char*>(dst) + at, static_cast<const char*>(src) + at, len, kind, streams[w]));
    }
    for (u32 w = 0; w < ways; ++w)
        HIP_TRY(hipStreamSynchronize(streams[w]));
    return CSA_OK;
}

} // namespace

extern "C" {

int csa_sort_partitions_u16(uint32_t count, const uint16_t* const* h_texts, const uint64_t* n, const uint64_t* index_base,
                            int key_words, uint8_t* const* h_sa40, csa_stats* stats)
{
    const char* who = "csa_sort_partitions_u16";
    if (count == 0)
        return CSA_OK;
    if (!h_texts || !n || !h_sa40)
        return fail(CSA_ERR_ARG, "%s: null list", who);
    u64 max_n = 0;
    for (u32 k = 0; k < count; ++k) {
        if (n[k] > CSA_MAX_PART_SZ)
            return fail(CSA_ERR_TOO_LARGE, "%s: partition %u has %llu suffixes, beyond the partition limit %llu", who, k,
                        (unsigned long long)n[k], (unsigned long long)CSA_MAX_PART_SZ);
        if (n[k] && (!h_texts[k] || !h_sa40[k]))
            return fail(CSA_ERR_ARG, "%s: partition %u has a null text or output pointer", who, k);
        const u64 base = index_base ? index_base[k] : 0;
        if (base > CSA_MAX_INDEX || base + n[k] > CSA_MAX_INDEX)
            return fail(CSA_ERR_TOO_LARGE, "%s: partition %u: suffix indices up to %llu do not fit 40 bits", who, k,
                        (unsigned long long)(base + n[k]));
        max_n = n[k] > max_n ? n[k] : max_n;
    }
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    csa_handle* h = nullptr;
    int rc = csa_create(max_n, key_words, &h);
    if (rc)
        return rc;
    // two sets of device buffers: while partition k is sorted out of one, k + 1 arrives in the other and k - 1 leaves it
    const u32 sets = count > 1 ? 2 : 1;
    u16* d_text[2] = {nullptr, nullptr};
    u8* d_sa[2] = {nullptr, nullptr};
    constexpr u32 WAYS = CSA_PIPELINE_COPY_WAYS, UP_WAYS = 1;
    hipStream_t st_up[UP_WAYS] = {}, st_sort = nullptr, st_down[WAYS] = {};
    hipError_t e = hipSuccess;
    for (u32 b = 0; b < sets && e == hipSuccess; ++b) {
        e = hipMalloc((void**)&d_text[b], max_n ? max_n * 2 : 4);
        if (e == hipSuccess)
            e = hipMalloc((void**)&d_sa[b], max_n ? max_n * 5 : 4);
    }
    // (all at the default priority)
    for (u32 w = 0; w < UP_WAYS; ++w)
        if (e == hipSuccess)
            e = hipStreamCreateWithFlags(&st_up[w], hipStreamNonBlocking);
    for (u32 w = 0; w < WAYS; ++w)
        if (e == hipSuccess)
            e = hipStreamCreateWithFlags(&st_down[w], hipStreamNonBlocking);
    if (e == hipSuccess)
        e = hipStreamCreateWithFlags(&st_sort, hipStreamNonBlocking);
    if (e != hipSuccess)
        rc = fail(CSA_ERR_HIP, "%s: %s while setting up buffers for %llu suffixes", who, hipGetErrorString(e), (unsigned long long)max_n);
    if (!rc) {
        HostPipeline pipe;
        std::thread uploader([&] {
            if (hipSetDevice(device) != hipSuccess) {
                fail(CSA_ERR_HIP, "%s: the upload thread cannot select device %d", who, device);
                return pipe.failed(CSA_ERR_HIP);
            }
            for (u32 k = 0; k < count; ++k) {
                // the buffer of partition k was last read by the sort of partition k - 2
                if (k >= 2 && !pipe.wait_for(pipe.sorted, k - 1))
                    return;
                const int c = copy_through(st_up, UP_WAYS, d_text[k % sets], h_texts[k], n[k] * 2, hipMemcpyHostToDevice);
                if (c)
                    return pipe.failed(c);
                pipe.advance(pipe.uploaded);
            }
        });
        std::thread downloader([&] {
            if (hipSetDevice(device) != hipSuccess) {
                fail(CSA_ERR_HIP, "%s: the download thread cannot select device %d", who, device);
                return pipe.failed(CSA_ERR_HIP);
            }
            for (u32 k = 0; k < count; ++k) {
                if (!pipe.wait_for(pipe.sorted, k + 1))
                    return;
                const int c = copy_through(st_down, WAYS, h_sa40[k], d_sa[k % sets], n[k] * 5, hipMemcpyDeviceToHost);
                if (c)
                    return pipe.failed(c);
                pipe.advance(pipe.downloaded);
            }
        });
        for (u32 k = 0; k < count; ++k) {
            // the text of partition k is in; the output buffer it writes to was last read by the download of partition k - 2
            if (!pipe.wait_for(pipe.uploaded, k + 1) || (k >= 2 && !pipe.wait_for(pipe.downloaded, k - 1)))
                break;
            const int c = csa_sort_partition_u16_dev(h, d_text[k % sets], n[k], index_base ? index_base[k] : 0, d_sa[k % sets], st_sort, 0,
                                                     stats ? &stats[k] : nullptr);
            if (c) {
                pipe.failed(c);
                break;
            }
            pipe.advance(pipe.sorted);
        }
        uploader.join();
        downloader.join();
        if (pipe.status != CSA_OK)
            rc = fail(pipe.status, "%s", pipe.message);
    }
    for (u32 w = 0; w < UP_WAYS; ++w)
        if (st_up[w])
            (void)hipStreamDestroy(st_up[w]);
    for (u32 w = 0; w < WAYS; ++w)
        if (st_down[w])
            (void)hipStreamDestroy(st_down[w]);
    if (st_sort)
        (void)hipStreamDestroy(st_sort);
    for (u32 b = 0; b < 2; ++b) {
        (void)hipFree(d_text[b]);
        (void)hipFree(d_sa[b]);
    }
    csa_destroy(h);
    return rc;
}

int csa_sort_partition_u16(const uint16_t* h_text, uint64_t n, int key_words, uint8_t* h_sa40, csa_stats* stats)
{
    if (n > CSA_MAX_PART_SZ)
        return fail(CSA_ERR_TOO_LARGE, "csa_sort_partition_u16: %llu suffixes exceed the partition limit %llu", (unsigned long long)n,
                    (unsigned long long)CSA_MAX_PART_SZ);
    if (n > 0 && (!h_text || !h_sa40))
        return fail(CSA_ERR_ARG, "csa_sort_partition_u16: null text or output pointer");
    if (stats) {
        memset(stats, 0, sizeof(*stats));
        stats->n = n;
        stats->key_words = key_words;
    }
    return csa_sort_partitions_u16(1, &h_text, &n, nullptr, key_words, &h_sa40, stats);
}

} // extern "C"
