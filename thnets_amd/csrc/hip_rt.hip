/*
 * Runtime plumbing of the engine: one stream, device memory, copies, events
 * and the per-launch profiler behind thhip_profile_*.
 */
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include "thhip_internal.h"

static hipStream_t g_stream;
static int g_init;

static void thhip_init_once(void)
{
	if (g_init)
		return;
	int n = 0;
	hipError_t rc = hipGetDeviceCount(&n);
	if (rc != hipSuccess || n < 1)
		THError("thnets HIP engine: no AMD GPU visible (hipGetDeviceCount: %s); this library has no CPU fallback",
			hipGetErrorString(rc));
	hipcheck(hipSetDevice(0));
	hipcheck(hipStreamCreate(&g_stream));
	g_init = 1;
}

hipStream_t thhip_stream(void)
{
	thhip_init_once();
	return g_stream;
}

extern "C" int thhip_device_count(void)
{
	int n = 0;
	if (hipGetDeviceCount(&n) != hipSuccess)
		return 0;
	return n;
}

extern "C" void *thhip_malloc(size_t bytes)
{
	void *p = 0;
	thhip_init_once();
	if (bytes == 0)
		bytes = 4;
	hipcheck(hipMalloc(&p, bytes));
	return p;
}

extern "C" void thhip_free(void *p)
{
	if (p)
		hipcheck(hipFree(p));
}

extern "C" void thhip_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, thhip_stream()));
	hipcheck(hipStreamSynchronize(thhip_stream()));
}

extern "C" void thhip_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, thhip_stream()));
	hipcheck(hipStreamSynchronize(thhip_stream()));
}

extern "C" void thhip_memcpy_d2d(void *dst, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, thhip_stream()));
}

__global__ void thhip_fill_bytes_kernel(unsigned char *p, int v, size_t n)
{
	size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	for (; i < n; i += (size_t)gridDim.x * blockDim.x)
		p[i] = (unsigned char)v;
}

extern "C" void thhip_memset(void *dst, int value, size_t bytes)
{
	if (!bytes)
		return;
	size_t blocks = (bytes + 255) / 256;
	if (blocks > 4096)
		blocks = 4096;
	thhip_fill_bytes_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>((unsigned char *)dst, value, bytes);
	hipcheck(hipGetLastError());
}

extern "C" void thhip_sync(void)
{
	hipcheck(hipStreamSynchronize(thhip_stream()));
}

/* ---- events ---- */
#define THHIP_NSLOTS 64
static hipEvent_t g_slots[THHIP_NSLOTS];

extern "C" void thhip_event_record(int slot)
{
	if (slot < 0 || slot >= THHIP_NSLOTS)
		THError("thhip_event_record: slot %d out of range", slot);
	if (!g_slots[slot])
		hipcheck(hipEventCreate(&g_slots[slot]));
	hipcheck(hipEventRecord(g_slots[slot], thhip_stream()));
}

extern "C" float thhip_event_ms(int a, int b)
{
	float ms = 0;
	if (a < 0 || a >= THHIP_NSLOTS || b < 0 || b >= THHIP_NSLOTS || !g_slots[a] || !g_slots[b])
		THError("thhip_event_ms: slots %d,%d not recorded", a, b);
	hipcheck(hipEventSynchronize(g_slots[b]));
	hipcheck(hipEventElapsedTime(&ms, g_slots[a], g_slots[b]));
	return ms;
}

/* ---- per-launch profiler ---- */
struct ProfRec { int family; hipEvent_t start, stop; double work; };
static std::vector<ProfRec> g_recs;
static std::vector<hipEvent_t> g_evpool;
static int g_prof_on;
static double g_fam_ms[THHIP_FAM_COUNT], g_fam_work[THHIP_FAM_COUNT];
static long g_fam_n[THHIP_FAM_COUNT];

static hipEvent_t prof_event(void)
{
	hipEvent_t e;
	if (!g_evpool.empty()) {
		e = g_evpool.back();
		g_evpool.pop_back();
		return e;
	}
	hipcheck(hipEventCreate(&e));
	return e;
}

static void prof_drain(void)
{
	if (g_recs.empty())
		return;
	hipcheck(hipStreamSynchronize(thhip_stream()));
	for (size_t i = 0; i < g_recs.size(); i++) {
		float ms = 0;
		hipcheck(hipEventElapsedTime(&ms, g_recs[i].start, g_recs[i].stop));
		g_fam_ms[g_recs[i].family] += ms;
		g_fam_work[g_recs[i].family] += g_recs[i].work;
		g_fam_n[g_recs[i].family]++;
		g_evpool.push_back(g_recs[i].start);
		g_evpool.push_back(g_recs[i].stop);
	}
	g_recs.clear();
}

int thhip_prof_begin(int family)
{
	/* 1: every family; otherwise the sum of 2 << family over the families wanted */
	/* a negative family: a launch that must not be bracketed (no events made) */
	if (family < 0 || !g_prof_on || (g_prof_on != 1 && !(g_prof_on & (2 << family))))
		return -1;
	if (g_recs.size() >= 4096)
		prof_drain();
	ProfRec r;
	r.family = family;
	r.start = prof_event();
	r.stop = prof_event();
	r.work = 0;
	hipcheck(hipEventRecord(r.start, thhip_stream()));
	g_recs.push_back(r);
	return (int)g_recs.size() - 1;
}

void thhip_prof_end(int token, double work)
{
	if (token < 0)
		return;
	g_recs[token].work = work;
	hipcheck(hipEventRecord(g_recs[token].stop, thhip_stream()));
}

extern "C" void thhip_profile_enable(int on)
{
	prof_drain();
	g_prof_on = on;
}

extern "C" void thhip_profile_reset(void)
{
	prof_drain();
	for (int i = 0; i < THHIP_FAM_COUNT; i++) {
		g_fam_ms[i] = g_fam_work[i] = 0;
		g_fam_n[i] = 0;
	}
}

extern "C" void thhip_profile_get(int family, double *ms, long *launches, double *work)
{
	prof_drain();
	if (family < 0 || family >= THHIP_FAM_COUNT)
		THError("thhip_profile_get: family %d out of range", family);
	*ms = g_fam_ms[family];
	*launches = g_fam_n[family];
	*work = g_fam_work[family];
}
