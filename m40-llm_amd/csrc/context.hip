// Context, memory, streams, events and graphs of the m40llm C ABI on HIP.
// Reference behaviour: cuda/kernels.cu:276-680, 1245-1292.
#include "common.hpp"

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <thread>

namespace {

constexpr size_t kGemmPackBytes = 8u << 20;      // 16 rows x K halves x 2 (hi, lo): K up to 128 Ki
constexpr size_t kAttnPartialBytes = 64u << 20;  // split-KV partials
constexpr size_t kSelectBytes = 8u << 20;        // block scores + selections

void free_scratch(M40StreamScratch& s) {
    if (s.gemm_pack) (void)hipFree(s.gemm_pack);
    if (s.attn_partial) (void)hipFree(s.attn_partial);
    if (s.select) (void)hipFree(s.select);
    if (s.tiled_pack) (void)hipFree(s.tiled_pack);
    if (s.attn_planes) (void)hipFree(s.attn_planes);
    s = M40StreamScratch{};
}

bool alloc_scratch(M40StreamScratch& s) {
    s = M40StreamScratch{};
    if (hipMalloc(&s.gemm_pack, kGemmPackBytes) != hipSuccess) return false;
    s.gemm_pack_bytes = kGemmPackBytes;
    if (hipMalloc(&s.attn_partial, kAttnPartialBytes) != hipSuccess) return false;
    s.attn_partial_bytes = kAttnPartialBytes;
    if (hipMalloc(&s.select, kSelectBytes) != hipSuccess) return false;
    s.select_bytes = kSelectBytes;
    return true;
}

// inv_freq[i] = base^(-2 i / head_dim) by the expression every rotating kernel uses when it has no table
__global__ void rope_table_kernel(float* table, uint32_t head_dim, float base) {
    const uint32_t i = threadIdx.x;
    if (i < head_dim / 2u) table[i] = m40_rope_inv_freq(i, head_dim, base);
}

}  // namespace

float4* m40_rope_cs_cache(M40llmCudaContext* ctx, const float* table) {
    if (!ctx || !table || !ctx->rope_tables || !ctx->rope_cs) return nullptr;
    return ctx->rope_cs + (table - ctx->rope_tables);
}

const float* m40_rope_inv_freq_table(M40llmCudaContext* ctx, uint32_t stream_kind, hipStream_t stream, uint32_t head_dim,
                                     float base) {
    if (!ctx || !ctx->rope_tables || stream_kind > 1u || head_dim / 2u > (uint32_t)kM40RopeTableLen || head_dim < 2u)
        return nullptr;
    float* tables = ctx->rope_tables + (size_t)stream_kind * kM40RopeSlots * kM40RopeTableLen;
    int free_slot = -1;
    for (int i = 0; i < kM40RopeSlots; ++i) {
        auto& slot = ctx->rope_slots[stream_kind][i];
        if (slot.ready && slot.head_dim == head_dim && slot.base == base) return tables + (size_t)i * kM40RopeTableLen;
        if (!slot.ready && free_slot < 0) free_slot = i;
    }
    if (free_slot < 0) return nullptr;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone) return nullptr;
    float* table = tables + (size_t)free_slot * kM40RopeTableLen;
    rope_table_kernel<<<1, kM40RopeTableLen, 0, stream>>>(table, head_dim, base);
    if (hipGetLastError() != hipSuccess) return nullptr;
    auto& slot = ctx->rope_slots[stream_kind][free_slot];
    slot.base = base; slot.head_dim = head_dim; slot.ready = 1u;
    return table;
}

extern "C" {

M40llmCudaContext* m40llm_create_context(int device_id) {
    // The reference auto-selects a Tesla M40 for device_id < 0 and falls back to
    // device 0 (kernels.cu:370-392); here every visible device is a gfx950, so a
    // negative id means device 0.
    int selected = device_id < 0 ? 0 : device_id;
    if (hipSetDevice(selected) != hipSuccess) return nullptr;

    M40llmCudaContext* ctx = new (std::nothrow) M40llmCudaContext();
    if (!ctx) return nullptr;
    std::memset(ctx, 0, sizeof(*ctx));
    ctx->device_id = selected;

    // Both streams keep the default priority: the prefill/decode split is kept for
    // ordering semantics only.
    if (hipStreamCreateWithFlags(&ctx->prefill_stream, hipStreamNonBlocking) != hipSuccess) {
        delete ctx;
        return nullptr;
    }
    if (hipStreamCreateWithFlags(&ctx->decode_stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipStreamDestroy(ctx->prefill_stream);
        delete ctx;
        return nullptr;
    }
    if (hipEventCreateWithFlags(&ctx->prefill_waits_decode_event, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&ctx->decode_waits_prefill_event, hipEventDisableTiming) != hipSuccess) {
        m40llm_destroy_context(ctx);
        return nullptr;
    }
    if (!alloc_scratch(ctx->scratch[0]) || !alloc_scratch(ctx->scratch[1])) {
        m40llm_destroy_context(ctx);
        return nullptr;
    }
    if (hipMalloc(&ctx->rope_tables, sizeof(float) * 2 * kM40RopeSlots * kM40RopeTableLen) != hipSuccess) {
        ctx->rope_tables = nullptr;
        m40llm_destroy_context(ctx);
        return nullptr;
    }
    const size_t cs_bytes = sizeof(float4) * 2 * kM40RopeSlots * kM40RopeTableLen;
    if (hipMalloc(reinterpret_cast<void**>(&ctx->rope_cs), cs_bytes) != hipSuccess || hipMemset(ctx->rope_cs, 0xff, cs_bytes) != hipSuccess) {
        m40llm_destroy_context(ctx);       // 0xff: no entry matches a position
        return nullptr;
    }
    if (hipHostMalloc(reinterpret_cast<void**>(&ctx->host_staging), sizeof(uint32_t) * kM40HostStagingWords, hipHostMallocDefault) != hipSuccess) {
        ctx->host_staging = nullptr;
        m40llm_destroy_context(ctx);
        return nullptr;
    }
    if (m40_attention_static_scratch_init(selected) != 0) {
        m40llm_destroy_context(ctx);
        return nullptr;
    }
    hipDeviceProp_t prop;
    ctx->num_cus = 256;
    if (hipGetDeviceProperties(&prop, selected) == hipSuccess && prop.multiProcessorCount > 0) {
        ctx->num_cus = prop.multiProcessorCount;
    }
    return ctx;
}

void m40llm_destroy_context(M40llmCudaContext* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device_id);
    if (ctx->decode_stream) (void)hipStreamSynchronize(ctx->decode_stream);
    if (ctx->prefill_stream) (void)hipStreamSynchronize(ctx->prefill_stream);
    free_scratch(ctx->scratch[0]);
    free_scratch(ctx->scratch[1]);
    if (ctx->rope_tables) (void)hipFree(ctx->rope_tables);
    if (ctx->rope_cs) (void)hipFree(ctx->rope_cs);
    if (ctx->host_staging) (void)hipHostFree(ctx->host_staging);
    if (ctx->prefill_waits_decode_event) (void)hipEventDestroy(ctx->prefill_waits_decode_event);
    if (ctx->decode_waits_prefill_event) (void)hipEventDestroy(ctx->decode_waits_prefill_event);
    if (ctx->prefill_stream) (void)hipStreamDestroy(ctx->prefill_stream);
    if (ctx->decode_stream) (void)hipStreamDestroy(ctx->decode_stream);
    delete ctx;
}

int m40llm_current_device_props(char* name_buf, size_t buf_len, int* major, int* minor, int* device_id) {
    if (!name_buf || buf_len == 0 || !major || !minor || !device_id) return -1;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -2;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return -3;
    size_t nlen = strnlen(prop.name, sizeof(prop.name));
    if (buf_len <= nlen) nlen = buf_len - 1;
    std::memcpy(name_buf, prop.name, nlen);
    name_buf[nlen] = '\0';
    *major = prop.major;
    *minor = prop.minor;
    *device_id = dev;
    return 0;
}

int m40llm_device_malloc(M40llmCudaContext* ctx, size_t bytes, void** out_ptr) {
    if (!ctx || !out_ptr) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    void* d = nullptr;
    if (hipMalloc(&d, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return -3;
    }
    *out_ptr = d;
    return 0;
}

int m40llm_device_free(M40llmCudaContext* ctx, void* ptr) {
    if (!ctx) return -1;
    if (!ptr) return 0;
    if (m40_ensure_device(ctx) != 0) return -3;
    if (hipFree(ptr) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
    }
    return 0;
}

int m40llm_memcpy_h2d(M40llmCudaContext* ctx, void* dst_device, const void* src_host, size_t bytes) {
    if (!ctx || !dst_device || !src_host) return -1;
    if (m40_ensure_device(ctx) != 0) return -3;
    if (hipMemcpy(dst_device, src_host, bytes, hipMemcpyHostToDevice) != hipSuccess) return -2;
    return 0;
}

int m40llm_memcpy_d2h(M40llmCudaContext* ctx, void* dst_host, const void* src_device, size_t bytes) {
    if (!ctx || !dst_host || !src_device) return -1;
    if (m40_ensure_device(ctx) != 0) return -3;
    if (hipMemcpy(dst_host, src_device, bytes, hipMemcpyDeviceToHost) != hipSuccess) return -2;
    return 0;
}

int m40llm_memcpy_d2d_async(M40llmCudaContext* ctx, void* dst_device, const void* src_device,
                            size_t bytes, uint32_t stream_kind) {
    if (!ctx || !dst_device || !src_device) return -1;
    if (m40_ensure_device(ctx) != 0) return -3;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -4;
    if (hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess) return -2;
    return 0;
}

int m40llm_validate_device_ptr(const void* ptr) {
    if (!ptr) return -1;
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
    }
    if (attr.type != hipMemoryTypeDevice) return -3;
    return 0;
}

int m40llm_upload_weights(M40llmCudaContext* ctx, const void* host_ptr, size_t num_bytes,
                          void** out_device_ptr) {
    if (!ctx || !host_ptr || !out_device_ptr) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    // The reference pins the caller's pages before the copy (kernels.cu:1276);
    // registering memory that already exists is not available on this platform, so
    // the copy runs from pageable memory.
    void* d_ptr = nullptr;
    if (hipMalloc(&d_ptr, num_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
    }
    if (hipMemcpy(d_ptr, host_ptr, num_bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(d_ptr);
        return -3;
    }
    *out_device_ptr = d_ptr;
    return 0;
}

// A byte range of a file into one new device allocation.  The range is read with positional reads into two
// pinned staging buffers by a few threads while the previous buffer's copy to the device is still in flight, so
// disk (or page cache) and the host-to-device link overlap; nothing the size of the file is ever held in host
// memory.  Replaces the reference's read-whole-file + upload_weights sequence (src/infer/load.rs:27-40,
// kernels.cu:1264-1290) for weight files.
int m40llm_ext_upload_file_range(M40llmCudaContext* ctx, const char* path, uint64_t file_offset, uint64_t num_bytes,
                                 void** out_device_ptr) {
    if (!ctx || !path || !out_device_ptr) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    const int fd = ::open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return -6;
    struct stat st {};
    if (::fstat(fd, &st) != 0 || st.st_size < 0 || file_offset > static_cast<uint64_t>(st.st_size) ||
        num_bytes > static_cast<uint64_t>(st.st_size) - file_offset) {
        ::close(fd);
        return -6;
    }
    constexpr uint64_t kStage = 16ull << 20;
    constexpr int kReaders = 8;
    void* d_ptr = nullptr;
    void* stage[2] = {nullptr, nullptr};
    hipEvent_t done[2] = {nullptr, nullptr};
    int rc = 0;
    if (hipMalloc(&d_ptr, num_bytes ? num_bytes : 4) != hipSuccess) {
        (void)hipGetLastError();
        ::close(fd);
        return -2;
    }
    const uint64_t stage_bytes = num_bytes < kStage ? (num_bytes ? num_bytes : 4) : kStage;
    for (int i = 0; i < 2 && rc == 0; ++i) {
        if (hipHostMalloc(&stage[i], stage_bytes, hipHostMallocDefault) != hipSuccess ||
            hipEventCreateWithFlags(&done[i], hipEventDisableTiming) != hipSuccess)
            rc = -2;
    }
    hipStream_t stream = ctx->prefill_stream;
    bool used[2] = {false, false};
    int which = 0;
    for (uint64_t at = 0; at < num_bytes && rc == 0; at += stage_bytes, which ^= 1) {
        const uint64_t n = num_bytes - at < stage_bytes ? num_bytes - at : stage_bytes;
        if (used[which] && hipEventSynchronize(done[which]) != hipSuccess) {
            rc = -3;
            break;
        }
        std::atomic<bool> short_read{false};
        auto read_part = [&](int part) {
            const uint64_t per = (n + kReaders - 1) / kReaders;
            uint64_t lo = per * part, hi = lo + per < n ? lo + per : n;
            while (lo < hi) {
                const ssize_t got = ::pread(fd, static_cast<char*>(stage[which]) + lo, hi - lo, static_cast<off_t>(file_offset + at + lo));
                if (got <= 0) {
                    if (got < 0 && errno == EINTR) continue;
                    short_read = true;
                    return;
                }
                lo += static_cast<uint64_t>(got);
            }
        };
        {
            std::thread readers[kReaders - 1];
            for (int t = 1; t < kReaders; ++t) readers[t - 1] = std::thread(read_part, t);
            read_part(0);
            for (auto& t : readers) t.join();
        }
        if (short_read) {
            rc = -6;
            break;
        }
        if (hipMemcpyAsync(static_cast<char*>(d_ptr) + at, stage[which], n, hipMemcpyHostToDevice, stream) != hipSuccess ||
            hipEventRecord(done[which], stream) != hipSuccess) {
            rc = -3;
            break;
        }
        used[which] = true;
    }
    if (hipStreamSynchronize(stream) != hipSuccess && rc == 0) rc = -3;
    for (int i = 0; i < 2; ++i) {
        if (done[i]) (void)hipEventDestroy(done[i]);
        if (stage[i]) (void)hipHostFree(stage[i]);
    }
    ::close(fd);
    if (rc != 0) {
        (void)hipFree(d_ptr);
        (void)hipGetLastError();
        return rc;
    }
    *out_device_ptr = d_ptr;
    return 0;
}

int m40llm_stream_synchronize(M40llmCudaContext* ctx, uint32_t stream_kind) {
    if (!ctx) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    if (hipStreamSynchronize(stream) != hipSuccess) return -4;
    return 0;
}

int m40llm_stream_wait_for_stream(M40llmCudaContext* ctx, uint32_t waiting_stream_kind,
                                  uint32_t signal_stream_kind) {
    if (!ctx) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t waiting = m40_select_stream(ctx, waiting_stream_kind);
    hipStream_t signal = m40_select_stream(ctx, signal_stream_kind);
    if (!waiting || !signal) return -3;
    hipEvent_t event = nullptr;
    if (waiting_stream_kind == 0 && signal_stream_kind == 1) {
        event = ctx->prefill_waits_decode_event;
    } else if (waiting_stream_kind == 1 && signal_stream_kind == 0) {
        event = ctx->decode_waits_prefill_event;
    } else if (waiting_stream_kind == signal_stream_kind) {
        return 0;
    }
    if (!event) return -4;
    if (hipEventRecord(event, signal) != hipSuccess) return -5;
    if (hipStreamWaitEvent(waiting, event, 0) != hipSuccess) return -6;
    return 0;
}

// ---- events -------------------------------------------------------------------
int m40llm_cuda_event_create(M40llmCudaContext* ctx, M40llmCudaEvent** out_event) {
    if (!ctx || !out_event) return -1;
    *out_event = nullptr;
    if (m40_ensure_device(ctx) != 0) return -2;
    M40llmCudaEvent* wrapped = new (std::nothrow) M40llmCudaEvent();
    if (!wrapped) return -3;
    wrapped->event = nullptr;
    if (hipEventCreate(&wrapped->event) != hipSuccess) {
        delete wrapped;
        return -3;
    }
    *out_event = wrapped;
    return 0;
}

int m40llm_cuda_event_record(M40llmCudaContext* ctx, M40llmCudaEvent* event, uint32_t stream_kind) {
    if (!ctx || !event || !event->event) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    return hipEventRecord(event->event, stream) == hipSuccess ? 0 : -4;
}

int m40llm_cuda_event_elapsed_sync(M40llmCudaContext* ctx, M40llmCudaEvent* start,
                                   M40llmCudaEvent* stop, float* elapsed_ms) {
    if (!ctx || !start || !stop || !start->event || !stop->event || !elapsed_ms) return -1;
    *elapsed_ms = 0.0f;
    if (m40_ensure_device(ctx) != 0) return -2;
    if (hipEventSynchronize(stop->event) != hipSuccess) return -3;
    return hipEventElapsedTime(elapsed_ms, start->event, stop->event) == hipSuccess ? 0 : -4;
}

void m40llm_cuda_event_destroy(M40llmCudaEvent* event) {
    if (!event) return;
    if (event->event) (void)hipEventDestroy(event->event);
    delete event;
}

// ---- graphs ---------------------------------------------------------------------
int m40llm_cuda_graph_begin_capture(M40llmCudaContext* ctx, uint32_t stream_kind) {
    if (!ctx) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    return hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed) == hipSuccess ? 0 : -4;
}

int m40llm_cuda_graph_end_capture(M40llmCudaContext* ctx, uint32_t stream_kind,
                                  M40llmCudaGraphExec** out_graph) {
    if (!ctx || !out_graph) return -1;
    *out_graph = nullptr;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    hipGraph_t graph = nullptr;
    if (hipStreamEndCapture(stream, &graph) != hipSuccess) {
        (void)hipGetLastError();
        return -4;
    }
    if (!graph) return -5;
    hipGraphExec_t exec = nullptr;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return -6;
    }
    M40llmCudaGraphExec* wrapped = new (std::nothrow) M40llmCudaGraphExec();
    if (!wrapped) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return -6;
    }
    wrapped->graph = graph;
    wrapped->exec = exec;
    *out_graph = wrapped;
    return 0;
}

int m40llm_cuda_graph_cancel_capture(M40llmCudaContext* ctx, uint32_t stream_kind) {
    if (!ctx) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    hipGraph_t graph = nullptr;
    hipError_t err = hipStreamEndCapture(stream, &graph);
    if (graph) (void)hipGraphDestroy(graph);
    if (err != hipSuccess) (void)hipGetLastError();
    return err == hipSuccess ? 0 : -4;
}

int m40llm_cuda_graph_launch(M40llmCudaContext* ctx, M40llmCudaGraphExec* graph, uint32_t stream_kind) {
    if (!ctx || !graph || !graph->exec) return -1;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    return hipGraphLaunch(graph->exec, stream) == hipSuccess ? 0 : -4;
}

int m40llm_cuda_graph_launch_timed_sync(M40llmCudaContext* ctx, M40llmCudaGraphExec* graph,
                                        uint32_t stream_kind, float* elapsed_ms) {
    if (!ctx || !graph || !graph->exec || !elapsed_ms) return -1;
    *elapsed_ms = 0.0f;
    if (m40_ensure_device(ctx) != 0) return -2;
    hipStream_t stream = m40_select_stream(ctx, stream_kind);
    if (!stream) return -3;
    hipEvent_t start = nullptr, stop = nullptr;
    if (hipEventCreate(&start) != hipSuccess) return -4;
    if (hipEventCreate(&stop) != hipSuccess) {
        (void)hipEventDestroy(start);
        return -5;
    }
    int rc = 0;
    if (hipEventRecord(start, stream) != hipSuccess) rc = -6;
    else if (hipGraphLaunch(graph->exec, stream) != hipSuccess) rc = -7;
    else if (hipEventRecord(stop, stream) != hipSuccess) rc = -8;
    else if (hipEventSynchronize(stop) != hipSuccess) rc = -9;
    else if (hipEventElapsedTime(elapsed_ms, start, stop) != hipSuccess) rc = -10;
    (void)hipEventDestroy(stop);
    (void)hipEventDestroy(start);
    return rc;
}

void m40llm_cuda_graph_destroy(M40llmCudaGraphExec* graph) {
    if (!graph) return;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

const char* m40llm_ext_build_info(void) {
    return "m40llm native: HIP gfx950 (wave64, MFMA f16 16x16x32), built " __DATE__;
}

}  // extern "C"
