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

/* (counts how often the stream was handed out: the profiler uses it to see that nothing was put on
 * the stream between two of its launches) */
static unsigned long g_stream_uses;
/* the profiler's open run of launches (below): anything else that asks for the stream ends it first */
static int g_prof_open = -1, g_prof_in_scope;
static void prof_close_run(void);

/* The batch window (below): a launch made while one is set, outside the code that honours it, is noted */
static int g_win_b0, g_win_n, g_win_scope, g_win_violated;

hipStream_t thhip_stream(void)
{
	thhip_init_once();
	if (g_prof_open >= 0 && !g_prof_in_scope)
		prof_close_run();
	if (g_win_n && !g_win_scope)
		g_win_violated = 1;
	++g_stream_uses;
	return g_stream;
}

/* ---- a window of the batch ----
 * THProcessFloat uploads a large batch in pieces and lets the first modules of the network run on the
 * images of a piece while the next one crosses the link.  Those modules run on the tensors of the whole
 * batch; while a window [b0, b0 + n) is set, the convolution entry points (conv_run, conv_mfma.hip) launch
 * their kernels on those images only.  Anything else that puts work on the stream while a window is set
 * would have processed the whole batch: it is noted, and the caller then runs the modules again on the
 * whole batch, without a window. */
extern "C" void thhip_batch_window(int b0, int n)
{
	g_win_b0 = b0;
	g_win_n = n > 0 ? n : 0;
	g_win_scope = 0;
}

extern "C" int thhip_batch_window_get(int *b0)
{
	*b0 = g_win_b0;
	return g_win_n;
}

extern "C" void thhip_batch_window_scope(int on)
{
	g_win_scope = on != 0;
}

extern "C" void thhip_batch_window_violate(void)
{
	g_win_violated = 1;
}

extern "C" int thhip_batch_window_violated(void)
{
	const int v = g_win_violated;
	g_win_violated = 0;
	return v;
}

extern "C" int thhip_device_count(void)
{
	int n = 0;
	if (hipGetDeviceCount(&n) != hipSuccess)
		return 0;
	return n;
}

/* How often this library has asked the runtime for something that allocates: device and
 * page-locked memory (taken or given back) and events.  A call that promises to allocate
 * nothing leaves it unchanged. */
static long g_alloc_calls;

extern "C" long thhip_alloc_calls(void)
{
	return g_alloc_calls;
}

extern "C" void *thhip_malloc(size_t bytes)
{
	void *p = 0;
	thhip_init_once();
	if (bytes == 0)
		bytes = 4;
	++g_alloc_calls;
	hipcheck(hipMalloc(&p, bytes));
	return p;
}

extern "C" void thhip_free(void *p)
{
	if (p) {
		++g_alloc_calls;
		hipcheck(hipFree(p));
	}
}

extern "C" void thhip_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, thhip_stream()));
	hipcheck(hipStreamSynchronize(thhip_stream()));
}

static void fault_check(void);

extern "C" void thhip_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, thhip_stream()));
	hipcheck(hipStreamSynchronize(thhip_stream()));
	fault_check();
}

/* Page-locked host memory: copies to and from it run at the link's rate and, queued with the
 * two calls below, return before they have finished. */
extern "C" void *thhip_host_malloc(size_t bytes)
{
	void *p = 0;
	thhip_init_once();
	++g_alloc_calls;
	hipcheck(hipHostMalloc(&p, bytes ? bytes : 4, hipHostMallocDefault));
	return p;
}

extern "C" void thhip_host_free(void *p)
{
	if (p) {
		++g_alloc_calls;
		hipcheck(hipHostFree(p));
	}
}

extern "C" void thhip_memcpy_h2d_async(void *dst, const void *src_pinned, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst, src_pinned, bytes, hipMemcpyHostToDevice, thhip_stream()));
}

extern "C" void thhip_memcpy_d2h_async(void *dst_pinned, const void *src, size_t bytes)
{
	hipcheck(hipMemcpyAsync(dst_pinned, src, bytes, hipMemcpyDeviceToHost, thhip_stream()));
}

/* Host -> device copies on a stream of their own, each followed by an event the engine's stream can be
 * made to wait for: a piece of a batch crosses the link while kernels work on the piece before it.  The
 * caller keeps the destination away from the engine's stream until that stream has waited for the event. */
#define THHIP_COPY_EVENTS 8
static hipStream_t g_copy_stream;
static hipEvent_t g_copy_events[THHIP_COPY_EVENTS];

extern "C" void thhip_memcpy_h2d_piece(void *dst, const void *src_pinned, size_t bytes, int event)
{
	thhip_init_once();
	if (event < 0 || event >= THHIP_COPY_EVENTS)
		THError("thhip_memcpy_h2d_piece: event %d out of range", event);
	if (!g_copy_stream) {
		++g_alloc_calls;
		hipcheck(hipStreamCreate(&g_copy_stream));
	}
	if (!g_copy_events[event]) {
		++g_alloc_calls;
		hipcheck(hipEventCreateWithFlags(&g_copy_events[event], hipEventDisableTiming));
	}
	hipcheck(hipMemcpyAsync(dst, src_pinned, bytes, hipMemcpyHostToDevice, g_copy_stream));
	hipcheck(hipEventRecord(g_copy_events[event], g_copy_stream));
}

extern "C" void thhip_wait_h2d_piece(int event)
{
	if (event < 0 || event >= THHIP_COPY_EVENTS || !g_copy_events[event])
		THError("thhip_wait_h2d_piece: event %d not recorded", event);
	hipcheck(hipStreamWaitEvent(thhip_stream(), g_copy_events[event], 0));
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
	fault_check();
}

/* ---- which XCD a workgroup runs on ----
 * The convolution kernels let the workgroups that compute the parts of one tile meet in their XCD's L2
 * (conv_xcd_last_arriver), which is right only if those workgroups -- all of one residue of blockIdx.x
 * modulo 8 -- run on one XCD.  The hardware hands workgroup b of a launch to XCD (b + r) % 8, with r fixed
 * for the launch (it changes when queues are created: measured on one stream, 0, then 7, 6, 5 as three more
 * streams were made).  Whether the GPU does so at all is checked here once per process on a grid of 4096
 * workgroups; that every launch did is checked by its own workgroups (conv_xcd_report), and a launch that
 * did not raises the flag below, which the next synchronisation turns into a repeat or an error. */
__global__ void xcd_probe_kernel(int *out)
{
	if (threadIdx.x == 0)
		out[blockIdx.x] = __builtin_amdgcn_s_getreg(THHIP_GETREG_XCC_ID);
}

/* 0x80000000 | r if workgroup b of the probe ran on XCD (b + r) % 8 for every b; 0 if not (then nothing
 * may rely on it). */
extern "C" unsigned thhip_xcd_map(void)
{
	static unsigned map;
	static int done;
	if (done)
		return map;
	const int n = 4096;
	int *dev = (int *)thhip_malloc(n * sizeof(int));
	std::vector<int> host(n);
	xcd_probe_kernel<<<dim3(n), dim3(64), 0, thhip_stream()>>>(dev);
	hipcheck(hipGetLastError());
	hipcheck(hipMemcpyAsync(host.data(), dev, n * sizeof(int), hipMemcpyDeviceToHost, thhip_stream()));
	hipcheck(hipStreamSynchronize(thhip_stream()));
	thhip_free(dev);
	bool ok = (unsigned)host[0] < 8u;
	for (int b = 0; b < n; b++)
		ok = ok && host[b] == ((host[0] + b) & 7);
	map = ok ? 0x80000000u | (unsigned)host[0] : 0;
	done = 1;
	return map;
}

/* One int in page-locked host memory that kernels set when they find themselves where they must not
 * be; thhip_sync and the copies to the host look at it. */
static int *g_fault;

extern "C" int *thhip_fault_flag(void)
{
	if (!g_fault) {
		g_fault = (int *)thhip_host_malloc(sizeof(int));
		*g_fault = 0;
	}
	return g_fault;
}

/* A caller that can run its work again (THProcessFloat, THProcessImages) holds the error back, asks
 * with thhip_fault_take() whether a kernel reported a fault meanwhile and, if so, repeats the forward
 * pass; everywhere else the report is fatal.  Either way the path that raised it is switched off first
 * (thhip_conv_parts_fault: the K parts of cut tiles go back to their second launch), so the repeat, or
 * the caller's next attempt, cannot meet it again. */
static int g_fault_hold, g_fault_seen;

extern "C" void thhip_fault_hold(int on)
{
	g_fault_hold = on != 0;
}

extern "C" int thhip_fault_take(void)
{
	const int code = g_fault_seen;
	g_fault_seen = 0;
	return code;
}

static void fault_check(void)
{
	if (!g_fault || !*(volatile int *)g_fault)
		return;
	const int code = *(volatile int *)g_fault;
	*g_fault = 0;
	thhip_conv_parts_fault();
	if (g_fault_hold) {
		g_fault_seen = code;
		return;
	}
	THError("thnets HIP engine: a kernel reported fault %d (1: the workgroups of a launch that share partial sums "
		"through their XCD's L2 were not handed to the XCDs in one order; the results since the last "
		"synchronisation are not valid.  The engine now adds such sums with a second launch, as after "
		"THHipSumPartsInKernel(0): run the forward pass again)", code);
}

/* ---- events ---- */
#define THHIP_NSLOTS 64
static hipEvent_t g_slots[THHIP_NSLOTS];

extern "C" void thhip_event_record(int slot)
{
	if (slot < 0 || slot >= THHIP_NSLOTS)
		THError("thhip_event_record: slot %d out of range", slot);
	if (!g_slots[slot]) {
		++g_alloc_calls;
		hipcheck(hipEventCreate(&g_slots[slot]));
	}
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
/* One record per run of launches of one family with nothing else on the stream between them: a start event
 * before the first, a stop event after the last (recorded when something else asks for the stream, or a
 * launch of another family begins).  No event sits between the launches of a run -- an event between two
 * dependent kernels costs 3-5 us of stream time, which showed on networks of short kernels -- so a
 * family's time is what its kernels take as the stream runs them, gaps between them included. */
struct ProfRec { int family; hipEvent_t start, stop; double work; bool shared_start; long n; };
static std::vector<ProfRec> g_recs;
static std::vector<hipEvent_t> g_evpool;
static int g_prof_on;
static double g_fam_ms[THHIP_FAM_COUNT], g_fam_work[THHIP_FAM_COUNT];
static long g_fam_n[THHIP_FAM_COUNT];

/* A run that follows another run with nothing put on the stream between them starts at that run's stop
 * event. */
static hipEvent_t g_last_stop;
static unsigned long g_last_stop_uses;	/* g_stream_uses right after that event was recorded; 0: none */

static hipEvent_t prof_event(void)
{
	hipEvent_t e;
	if (!g_evpool.empty()) {
		e = g_evpool.back();
		g_evpool.pop_back();
		return e;
	}
	++g_alloc_calls;
	hipcheck(hipEventCreate(&e));
	return e;
}

static void prof_close_run(void)
{
	if (g_prof_open < 0)
		return;
	ProfRec &r = g_recs[g_prof_open];
	hipcheck(hipEventRecord(r.stop, g_stream));
	g_last_stop = r.stop;
	g_last_stop_uses = g_stream_uses;
	g_prof_open = -1;
}

static void prof_drain(void)
{
	prof_close_run();
	if (g_recs.empty())
		return;
	hipcheck(hipStreamSynchronize(thhip_stream()));
	for (size_t i = 0; i < g_recs.size(); i++) {
		float ms = 0;
		hipcheck(hipEventElapsedTime(&ms, g_recs[i].start, g_recs[i].stop));
		g_fam_ms[g_recs[i].family] += ms;
		g_fam_work[g_recs[i].family] += g_recs[i].work;
		g_fam_n[g_recs[i].family] += g_recs[i].n;
		if (!g_recs[i].shared_start)
			g_evpool.push_back(g_recs[i].start);
		g_evpool.push_back(g_recs[i].stop);
	}
	g_recs.clear();
	g_last_stop_uses = 0;
}

int thhip_prof_begin(int family)
{
	/* 1: every family; otherwise the sum of 2 << family over the families wanted */
	/* a negative family: a launch that must not be bracketed (no events made) */
	if (family < 0 || !g_prof_on || (g_prof_on != 1 && !(g_prof_on & (2 << family))))
		return -1;
	if (g_prof_in_scope)
		return -1;	/* (a bracket inside a bracket is part of the outer one) */
	if (g_prof_open >= 0 && g_recs[g_prof_open].family == family) {
		/* the run goes on (anything else on the stream since its last launch would have closed it) */
		g_recs[g_prof_open].n++;
		g_prof_in_scope = 1;
		return g_prof_open;
	}
	prof_close_run();
	if (g_recs.size() >= 4096)
		prof_drain();
	ProfRec r;
	r.family = family;
	r.shared_start = g_last_stop_uses && g_last_stop_uses == g_stream_uses;
	if (r.shared_start)
		r.start = g_last_stop;
	else {
		r.start = prof_event();
		hipcheck(hipEventRecord(r.start, thhip_stream()));
	}
	r.stop = prof_event();
	r.work = 0;
	r.n = 1;
	g_recs.push_back(r);
	g_prof_in_scope = 1;
	return (int)g_recs.size() - 1;
}

void thhip_prof_end(int token, double work)
{
	if (token < 0)
		return;
	g_recs[token].work += work;
	g_prof_in_scope = 0;
	g_prof_open = token;	/* its stop event: when the run ends */
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

/* ---- what the matrix cores sustain from registers alone ----
 * A loop of MFMAs on four independent accumulators, operands in registers (random values), no
 * memory traffic: the rate a convolution kernel could reach if everything else were free.
 * `waves_per_simd` workgroups of four wavefronts per CU (1..8) are resident for the whole run.
 * Measured on one MI355X: fp32 32x32x2 reaches 154 TFLOP/s with one or two wavefronts per SIMD
 * but 117 with three and 87-101 with four and more; fp16 32x32x16 1.64-1.71 PFLOP/s and int8
 * 32x32x32 3.5-3.7 POP/s with random operands once the loop has run for half a second (1.2
 * PFLOP/s over its first 40 ms), 2.48 PFLOP/s and 4.96 POP/s with all-zero operands: the
 * half and 8-bit rates are set by the power the operands' bit activity draws. */
template <int DT>
__global__ __launch_bounds__(256) void mfma_probe_kernel(float *out, const float *in, int iters)
{
	float s = 0;
	if constexpr (DT == THHIP_F32) {
		floatx16 acc[4];
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				acc[i][r] = 0;
		float a[8], b[8];
		for (int u = 0; u < 8; u++) {
			a[u] = in[(threadIdx.x * 8 + u) & 4095];
			b[u] = in[(threadIdx.x * 8 + u + 1777) & 4095];
		}
		for (int it = 0; it < iters; it++) {
#pragma unroll
			for (int u = 0; u < 8; u++)
#pragma unroll
				for (int i = 0; i < 4; i++)
					acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc[i], 0, 0, 0);
		}
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				s += acc[i][r];
	} else if constexpr (DT == THHIP_F16) {
		floatx16 acc[4];
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				acc[i][r] = 0;
		halfx8 a[8], b[8];
		for (int u = 0; u < 8; u++)
			for (int e = 0; e < 8; e++) {
				a[u][e] = (_Float16)in[(threadIdx.x * 8 + u + 3 * e) & 4095];
				b[u][e] = (_Float16)in[(threadIdx.x * 8 + u + 1777 + 5 * e) & 4095];
			}
		for (int it = 0; it < iters; it++) {
#pragma unroll
			for (int u = 0; u < 8; u++)
#pragma unroll
				for (int i = 0; i < 4; i++)
					acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[u], b[u], acc[i], 0, 0, 0);
		}
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				s += acc[i][r];
	} else {
		intx16 acc[4];
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				acc[i][r] = 0;
		intx4 a[8], b[8];
		for (int u = 0; u < 8; u++)
			for (int e = 0; e < 4; e++) {
				a[u][e] = (int)(in[(threadIdx.x * 8 + u + 3 * e) & 4095] * 2e9f);
				b[u][e] = (int)(in[(threadIdx.x * 8 + u + 1777 + 5 * e) & 4095] * 2e9f);
			}
		for (int it = 0; it < iters; it++) {
#pragma unroll
			for (int u = 0; u < 8; u++)
#pragma unroll
				for (int i = 0; i < 4; i++)
					acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u], b[u], acc[i], 0, 0, 0);
		}
		for (int i = 0; i < 4; i++)
			for (int r = 0; r < 16; r++)
				s += (float)acc[i][r];
	}
	out[blockIdx.x * 256 + threadIdx.x] = s;
}

/* Runs the loop above for about `ms` milliseconds and returns the rate in operations per
 * second (2 per multiply-add); dtype THHIP_F32, THHIP_F16 or THHIP_U8 (signed 8-bit operands). */
extern "C" double thhip_probe_mfma(int dtype, int waves_per_simd, double ms)
{
	if (waves_per_simd < 1 || waves_per_simd > 8 || ms <= 0 || (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_U8))
		THError("thhip_probe_mfma(%d, %d, %g): dtype fp32 / fp16 / uint8, 1 to 8 wavefronts per SIMD", dtype, waves_per_simd, ms);
	thhip_init_once();
	int dev, cus;
	hipcheck(hipGetDevice(&dev));
	hipcheck(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
	const int blocks = cus * waves_per_simd;
	float host[4096];
	unsigned long long st = 88172645463325252ull;
	for (int i = 0; i < 4096; i++) {	/* xorshift64: uniform in [-1, 1) */
		st ^= st << 13;
		st ^= st >> 7;
		st ^= st << 17;
		host[i] = (float)((double)(st >> 11) / 9007199254740992.0 * 2.0 - 1.0);
	}
	float *in = (float *)thhip_malloc(sizeof(host)), *out = (float *)thhip_malloc((size_t)blocks * 256 * sizeof(float));
	thhip_memcpy_h2d(in, host, sizeof(host));
	const double per_mfma = dtype == THHIP_F32 ? 4096.0 : dtype == THHIP_F16 ? 32768.0 : 65536.0;
	hipEvent_t e0, e1;
	++g_alloc_calls;
	hipcheck(hipEventCreate(&e0));
	++g_alloc_calls;
	hipcheck(hipEventCreate(&e1));
	double rate = 0;
	int iters = 64;
	for (int pass = 0; pass < 2; pass++) {	/* a short run sizes the long one */
		/* (through thhip_stream(), so that the profiler sees the stream in use and starts
		 * the next profiled launch at an event of its own) */
		hipcheck(hipEventRecord(e0, thhip_stream()));
		if (dtype == THHIP_F32)
			mfma_probe_kernel<THHIP_F32><<<dim3(blocks), dim3(256), 0, thhip_stream()>>>(out, in, iters);
		else if (dtype == THHIP_F16)
			mfma_probe_kernel<THHIP_F16><<<dim3(blocks), dim3(256), 0, thhip_stream()>>>(out, in, iters);
		else
			mfma_probe_kernel<THHIP_U8><<<dim3(blocks), dim3(256), 0, thhip_stream()>>>(out, in, iters);
		hipcheck(hipGetLastError());
		hipcheck(hipEventRecord(e1, thhip_stream()));
		hipcheck(hipEventSynchronize(e1));
		float t;
		hipcheck(hipEventElapsedTime(&t, e0, e1));
		rate = (double)blocks * 4 * iters * 32 * per_mfma / (t * 1e-3);
		if (pass == 0) {
			const double want = ms / (t > 1e-3 ? t : 1e-3) * iters;
			iters = want > 5e7 ? 50000000 : want < 64 ? 64 : (int)want;
		}
	}
	hipcheck(hipEventDestroy(e0));
	hipcheck(hipEventDestroy(e1));
	thhip_free(in);
	thhip_free(out);
	return rate;
}
