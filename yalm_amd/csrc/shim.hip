// shim.hip — the device shim of the C ABI (include/yalm_hip.h): thread-local errors,
// device selection, memory, streams and the synthetic initialiser. Replaces
// /root/reference/src/infer.cu:33-90. Every engine library links this unit.
#include "../../include/yalm_hip.h"

#include <hip/hip_runtime.h>

#include <string>

#include "decoder.h"
#include "device_common.h"

// ------------------------------------------------------------------ errors
static thread_local std::string g_err;

void set_err(const std::string &s) {
	g_err = s;
}

extern "C" const char *yalm_last_error(void) {
	return g_err.c_str();
}

// ------------------------------------------------------------------ shim
extern "C" int yalm_set_device(int device) {
	HIPCHK(hipSetDevice(device));
	return YALM_OK;
}

extern "C" void *yalm_upload(const void *host, size_t size) {
	void *dev = nullptr;
	if (hipMalloc(&dev, size ? size : 1) != hipSuccess) {
		set_err("hipMalloc failed in yalm_upload");
		return nullptr;
	}
	if (size && hipMemcpy(dev, host, size, hipMemcpyHostToDevice) != hipSuccess) {
		set_err("hipMemcpy H2D failed in yalm_upload");
		(void)hipFree(dev);
		return nullptr;
	}
	return dev;
}

extern "C" void *yalm_alloc(size_t size) {
	void *dev = nullptr;
	if (hipMalloc(&dev, size ? size : 1) != hipSuccess) {
		set_err("hipMalloc failed in yalm_alloc");
		return nullptr;
	}
	if (hipMemset(dev, 0, size ? size : 1) != hipSuccess) {
		set_err("hipMemset failed in yalm_alloc");
		(void)hipFree(dev);
		return nullptr;
	}
	return dev;
}

extern "C" int yalm_download(void *host, const void *device, size_t size) {
	HIPCHK(hipMemcpy(host, device, size, hipMemcpyDeviceToHost));
	return YALM_OK;
}

extern "C" int yalm_register_host(void *host, size_t size) {
	// some hosts refuse to pin memory that already exists; the error must not stay behind
	// for the next HIP call to report
	const hipError_t e = hipHostRegister(host, size, hipHostRegisterDefault);
	if (e != hipSuccess) {
		(void)hipGetLastError();
		set_err(std::string("hipHostRegister failed: ") + hipGetErrorString(e));
		return YALM_ERR_HIP;
	}
	return YALM_OK;
}

extern "C" int yalm_unregister_host(void *host) {
	HIPCHK(hipHostUnregister(host));
	return YALM_OK;
}

extern "C" int yalm_free(void *device) {
	HIPCHK(hipFree(device));
	return YALM_OK;
}

extern "C" int yalm_stream_create(yalm_stream *out) {
	ARGCHK(out, "null stream out");
	hipStream_t s;
	HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
	*out = reinterpret_cast<yalm_stream>(s);
	return YALM_OK;
}

// A stream restricted to CU block `part` of `n_parts` (hipExtStreamCreateWithCUMask):
// bits [part * ncu / n_parts, (part + 1) * ncu / n_parts). The driver spreads such a block
// evenly over the 8 XCDs (tools/cumask_probe.hip, profiles/r6a_cumask_probe.txt: 256 / N CUs
// on all 8 XCCs, disjoint between parts); an interleaved mask (bit i to part i mod N) was
// not honoured (every part ran on all 256 CUs). Used to run N tensor-parallel rank
// processes on ONE GPU as N disjoint sets of CUs (the multi-GPU rehearsal).
extern "C" int yalm_stream_create_cu_part(int part, int n_parts, yalm_stream *out) {
	ARGCHK(out && n_parts >= 1 && part >= 0 && part < n_parts, "yalm_stream_create_cu_part: bad argument");
	const int ncu = device_cu_count();
	ARGCHK(ncu % n_parts == 0 && ncu <= 32 * YALM_CU_MASK_WORDS, "yalm_stream_create_cu_part: CUs do not divide");
	uint32_t m[YALM_CU_MASK_WORDS] = {};
	for (int i = part * (ncu / n_parts); i < (part + 1) * (ncu / n_parts); ++i)
		m[i / 32] |= 1u << (i % 32);
	hipStream_t s;
	HIPCHK(hipExtStreamCreateWithCUMask(&s, (uint32_t)((ncu + 31) / 32), m));
	*out = reinterpret_cast<yalm_stream>(s);
	return YALM_OK;
}

extern "C" int yalm_stream_destroy(yalm_stream s) {
	HIPCHK(hipStreamDestroy(reinterpret_cast<hipStream_t>(s)));
	return YALM_OK;
}

extern "C" int yalm_stream_sync(yalm_stream s) {
	HIPCHK(hipStreamSynchronize(reinterpret_cast<hipStream_t>(s)));
	return YALM_OK;
}

// Deterministic synthetic initialiser — the same integer hash as the CPU
// oracle (oracle/yalm_oracle.c orc_synth_*), so a random-weight model of a
// real shape can be built in HBM and reproduced bit-exactly on the host.
__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
	x += 0x9E3779B97F4A7C15ull;
	x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
	x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
	return x ^ (x >> 31);
}

__global__ void synth_kernel(void *dst, size_t n, int dtype, uint64_t seed, float scale, float offset) {
	const float k = scale * (1.0f / 8388608.0f);
	for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
		uint64_t h = splitmix64(seed ^ ((uint64_t)i * 0xD1B54A32D192ED03ull));
		int32_t s = (int32_t)(h >> 40) - 8388608;
		if (dtype == 0) {
			((float *)dst)[i] = __builtin_fmaf((float)s, k, offset);
		} else {
			float v = __fmul_rn((float)s, k);
			uint32_t hb = f2h(v); // f2h keeps the f32 rounding step (no fma_mix fusion)
			if (dtype == 2) { // bf16: round to nearest even on the f32 bits
				const uint32_t u = __builtin_bit_cast(uint32_t, v);
				((uint16_t *)dst)[i] = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
			} else if (dtype == 1)
				((uint16_t *)dst)[i] = (uint16_t)hb;
			else
				((uint8_t *)dst)[i] = (uint8_t)((hb + 0x7Fu + ((hb >> 8) & 1u)) >> 8);
		}
	}
}

extern "C" int yalm_synth(void *device, size_t n, int dtype, uint64_t seed, float scale, float offset, yalm_stream s) {
	ARGCHK(dtype == YALM_F32 || dtype == YALM_F16 || dtype == YALM_BF16 || dtype == YALM_F8E5M2, "yalm_synth: bad dtype");
	hipStream_t st = reinterpret_cast<hipStream_t>(s);
	synth_kernel<<<4096, 256, 0, st>>>(device, n, dtype, seed, scale, offset);
	HIPCHK(hipGetLastError());
	return YALM_OK;
}

int device_cu_count() {
	static int n = 0;
	if (!n) {
		int dev = 0;
		if (hipGetDevice(&dev) != hipSuccess ||
		    hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
			n = 256;
	}
	return n;
}

