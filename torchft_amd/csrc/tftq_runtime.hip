// Device selection and the small-copy helper of the C ABI: tftq_check_device,
// tftq_upload_pointers and tftq_put_bytes.

#include <string.h>

#include "tftq_device.h"

// 3584 bytes of payload per launch: with the two other arguments the kernel's
// argument block stays below the 4 KB that a launch can carry.
constexpr int PUT_WORDS = 448;
struct PutChunk {
    uint64_t w[PUT_WORDS];
};

__global__ __launch_bounds__(TFTQ_WG) void k_put(uint64_t *dst, int n, const PutChunk c)
{
    for (int i = (int)threadIdx.x; i < n; i += TFTQ_WG) dst[i] = c.w[i];
}

int tftq_put_bytes(void *dst_device, const void *src_host, size_t bytes, hipStream_t st)
{
    if (bytes == 0) return 0;
    if (!dst_device || !src_host || (bytes & 7) != 0 || ((uintptr_t)dst_device & 7) != 0) return TFTQ_E_ARG;
    const size_t words = bytes / 8;
    PutChunk c;
    for (size_t done = 0; done < words; done += PUT_WORDS) {
        const int n = (int)(words - done < (size_t)PUT_WORDS ? words - done : (size_t)PUT_WORDS);
        memcpy(c.w, (const uint8_t *)src_host + done * 8, (size_t)n * 8);
        uint64_t *dst = (uint64_t *)dst_device + done;
        void *args[3] = {(void *)&dst, (void *)&n, (void *)&c};
        const hipError_t e = hipLaunchKernel((const void *)k_put, dim3(1), dim3(TFTQ_WG), args, 0, st);
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

extern "C" int tftq_upload_pointers(const tftq_plan *plan, const void *const *tensors, void *pointers, int device,
                                    void *stream)
{
    if (!plan || !tensors || !pointers) return TFTQ_E_ARG;
    DeviceScope scope(device);
    if (scope.err != hipSuccess) return (int)scope.err;
    return tftq_put_bytes(pointers, tensors, (size_t)plan->nseg * 8, (hipStream_t)stream);
}

extern "C" int tftq_check_device(int device)
{
    int dev = device;
    hipError_t e = hipSuccess;
    if (dev < 0) e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    const char *a = prop.gcnArchName;
    if (!(a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0')) return TFTQ_E_ARCH;
    DeviceScope scope(dev);
    if (scope.err != hipSuccess) return (int)scope.err;
    return tftq_static_table_setup();
}
