// What a DevicePlugin adapter inside the reference's engine would hand to this library, built
// WITHOUT this repository's loader: the structs below are declared here with the field order of
// the reference's own headers (csrc/plugins/cuda/kernel/proxy_trigger.h:8-30 for the two trigger
// handles and the 32-byte union, include/engine/ring_buffer.h:8-11 for the raw trigger,
// include/engine/primitive.h:8-17 for PrimitiveMeta), filled by hand for the two-rank bf16 ring
// allreduce of 2048 elements (chunk 1024; per rank: notify 100, wait 100, reduce, notify 0, wait 0,
// copy, notify 0, wait 0 - primitive ids cuda_reduce_bf16 = 3, cuda_copy_bf16 = 8,
// cuda_wait_notify = 21, cuda_notify = 22, csrc/plugins/cuda/kernel/primitive_config.h:11-34), and
// passed to pccl_hip_register_triggers as raw memory.  The library's own pccl_trigger /
// pccl_primitive_meta are only named in the two casts.  Then the reference's closed form (tests/
// test_correctness.py:142,170-171): every element of rank r is r + 1, every element of the result
// is R (R + 1) / 2 = 3.
//
// usage: adapter_check          exit status 0 and a line "ok ..." on success
#include <hip/hip_runtime_api.h>
#include <pccl_hip.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

namespace reference_layout {

struct ProxyTrigger { uint64_t raw[4]; };
struct OpProxyTriggerCudaHandle { char primitive_type; int op_index; int peer_rank; int offset_0; int offset_1; int offset_2; int size; };
struct SignalProxyTriggerCudaHandle { char primitive_type; int op_index; int peer_rank; int offset; int participants; };
union op { ProxyTrigger raw; OpProxyTriggerCudaHandle op_handle; SignalProxyTriggerCudaHandle signal_handle; };
struct PrimitiveMeta {
    int op_seq_index_;
    int num_next_ops_;
    int num_dependencies_;
    int next_primitive_index[8];
    int device_type;
    int channel;
    uint64_t params[4];
};

}  // namespace reference_layout

using namespace reference_layout;
static_assert(sizeof(op) == 32 && sizeof(op) == sizeof(pccl_trigger), "a trigger is 32 bytes on both sides");
static_assert(sizeof(PrimitiveMeta) == 88 && sizeof(PrimitiveMeta) == sizeof(pccl_primitive_meta), "PrimitiveMeta is 88 bytes on both sides");

static op signal(char type, int index, int peer, int id) {
    op t;
    std::memset(&t, 0, sizeof(t));
    t.signal_handle.primitive_type = type; t.signal_handle.op_index = index; t.signal_handle.peer_rank = peer;
    t.signal_handle.offset = id; t.signal_handle.participants = 0;
    return t;
}

static op data(char type, int index, int peer, int off0, int off1, int off2, int size) {
    op t;
    std::memset(&t, 0, sizeof(t));
    t.op_handle.primitive_type = type; t.op_handle.op_index = index; t.op_handle.peer_rank = peer;
    t.op_handle.offset_0 = off0; t.op_handle.offset_1 = off1; t.op_handle.offset_2 = off2; t.op_handle.size = size;
    return t;
}

static uint16_t bf16_of_small_int(int v) {
    float f = (float)v;
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}

#define HIP_OK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_)); return 1; } } while (0)
#define PCCL_OK_(expr) do { if ((expr) < 0) { std::fprintf(stderr, "%s: %s\n", #expr, pccl_hip_last_error()); return 1; } } while (0)

int main() {
    const int R = 2, N = 2048, chunk = N / R;
    const char kReduceBf16 = 3, kCopyBf16 = 8, kWait = 21, kNotify = 22;
    pccl_hip_ctx* ctx = nullptr;
    PCCL_OK_(pccl_hip_create(&ctx, 0, R));
    for (int rank = 0; rank < R; ++rank) {
        const int other = 1 - rank;
        // rank r reduces chunk (r - 1) mod 2 from the other rank, then copies chunk r from it
        const int red = ((rank + R - 1) % R) * chunk, cpy = rank * chunk;
        std::vector<op> trig = {
            signal(kNotify, 0, other, 100), signal(kWait, 1, other, 100),
            data(kReduceBf16, 2, other, red, red, red, chunk),
            signal(kNotify, 3, other, 0), signal(kWait, 4, other, 0),
            data(kCopyBf16, 5, other, cpy, cpy, 0, chunk),
            signal(kNotify, 6, other, 0), signal(kWait, 7, other, 0),
        };
        std::vector<PrimitiveMeta> meta(trig.size());
        for (size_t i = 0; i < meta.size(); ++i) {       // one linear chain on channel 0
            PrimitiveMeta& m = meta[i];
            std::memset(&m, 0, sizeof(m));
            m.op_seq_index_ = (int)i;
            m.num_dependencies_ = i == 0 ? 0 : 1;
            m.num_next_ops_ = i + 1 < meta.size() ? 1 : 0;
            if (m.num_next_ops_) m.next_primitive_index[0] = (int)i + 1;
            m.device_type = 1;
            m.channel = 0;
            std::memcpy(m.params, &trig[i], sizeof(m.params));
        }
        PCCL_OK_(pccl_hip_register_triggers(ctx, "ring2", rank, reinterpret_cast<const pccl_trigger*>(trig.data()),
                                            reinterpret_cast<const pccl_primitive_meta*>(meta.data()), (int)trig.size(), "allreduce"));
    }
    pccl_program_info info;
    PCCL_OK_(pccl_hip_op_info(ctx, "ring2", &info));
    if (info.num_data_ops != 4 || info.dtype != PCCL_BF16 || info.residual_signals != 0 || info.algorithmic_bytes != 5 * (R - 1) * N * 2) {
        std::fprintf(stderr, "linked program: %d data ops, dtype %d, %d residual signals, %lld algorithmic bytes\n", info.num_data_ops,
                     info.dtype, info.residual_signals, (long long)info.algorithmic_bytes);
        return 1;
    }
    void *in[R], *out[R];
    std::vector<uint16_t> host(N);
    for (int r = 0; r < R; ++r) {
        HIP_OK(hipMalloc(&in[r], N * 2));
        HIP_OK(hipMalloc(&out[r], N * 2));
        for (int i = 0; i < N; ++i) host[i] = bf16_of_small_int(r + 1);
        HIP_OK(hipMemcpy(in[r], host.data(), N * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemset(out[r], 0, N * 2));
    }
    const char* modes[] = {"auto", "stepwise", "persistent"};
    for (const char* mode : modes) {
        PCCL_OK_(pccl_hip_set_option(ctx, "mode", mode));
        for (int r = 0; r < R; ++r) HIP_OK(hipMemset(out[r], 0, N * 2));
        PCCL_OK_(pccl_hip_execute(ctx, "ring2", in, out, N * 2, N * 2, nullptr, 1));
        for (int r = 0; r < R; ++r) {
            HIP_OK(hipMemcpy(host.data(), out[r], N * 2, hipMemcpyDeviceToHost));
            for (int i = 0; i < N; ++i)
                if (host[i] != bf16_of_small_int(R * (R + 1) / 2)) {
                    std::fprintf(stderr, "mode %s: rank %d element %d is 0x%04x, expected 0x%04x\n", mode, r, i, host[i], bf16_of_small_int(3));
                    return 1;
                }
        }
    }
    for (int r = 0; r < R; ++r) { HIP_OK(hipFree(in[r])); HIP_OK(hipFree(out[r])); }
    PCCL_OK_(pccl_hip_destroy(ctx));
    std::printf("ok triggers laid out by the reference's headers: ranks=%d elements=%d result=%d\n", R, N, R * (R + 1) / 2);
    return 0;
}
