/*
 * Host-side tensor bookkeeping with the semantics of the reference's
 * thbasic.c:17-460 (reference-counted storages, <= 4 dimensions, strides in
 * elements).  Only what the engine glue needs is here; all arithmetic lives in
 * the HIP kernels.  A storage whose mustfree is TH_MUSTFREE_HIP owns device
 * memory and is released with thhip_free.
 */
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "th_engine.h"

/* thbasic.c:172-181: fatal, message on stderr, exit(-1). */
void THError(const char *fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vfprintf(stderr, fmt, ap);
	va_end(ap);
	fputc('\n', stderr);
	fflush(stderr);
	exit(-1);
}

static void *xmalloc(size_t n)
{
	void *p = malloc(n ? n : 1);
	if (!p)
		THError("Out of memory trying to allocate %zu bytes", n);
	return p;
}

THFloatStorage *THFloatStorage_new(long size)
{
	THFloatStorage *s = xmalloc(sizeof(*s));
	s->data = xmalloc(sizeof(float) * (size_t)size);
	s->nref = 1;
	s->mustfree = 1;
	return s;
}

THFloatStorage *THFloatStorage_newwithbuffer(void *buffer)
{
	THFloatStorage *s = xmalloc(sizeof(*s));
	s->data = buffer;
	s->nref = 1;
	s->mustfree = 0;
	return s;
}

THFloatTensor *THFloatTensor_new(void)
{
	return calloc(1, sizeof(THFloatTensor));
}

void THFloatTensor_free(THFloatTensor *t)
{
	if (!t)
		return;
	if (t->storage)
		thhip_storage_release(t->storage);
	free(t);
}

long THFloatTensor_nElement(THFloatTensor *t)
{
	long n = 1;
	if (t->nDimension == 0)
		return 0;
	for (int i = 0; i < t->nDimension; i++)
		n *= t->size[i];
	return n;
}

float *THFloatTensor_data(THFloatTensor *t)
{
	if (t && t->storage && t->storage->data)
		return t->storage->data + t->storageOffset;
	return 0;
}

/* Contiguous row-major shape; host storages are (re)allocated when the
 * element count changes (thbasic.c:58-168). */
void THFloatTensor_resize(THFloatTensor *t, long *size, int nDimension)
{
	long before = THFloatTensor_nElement(t), stride = 1;
	int unsized = 0;
	t->nDimension = nDimension;
	for (int i = nDimension - 1; i >= 0; i--) {
		t->size[i] = size[i];
		t->stride[i] = stride;
		stride *= size[i];
		if (size[i] == -1)
			unsized = 1;
	}
	if (before == THFloatTensor_nElement(t))
		return;
	if (unsized) {
		if (t->storage) {
			thhip_storage_release(t->storage);
			t->storage = 0;
		}
		return;
	}
	if (!t->storage)
		t->storage = THFloatStorage_new(stride);
	else if (TH_IS_HIP_STORAGE(t->storage->mustfree))
		THError("Resizing of device tensors is done by the engine, not by THFloatTensor_resize");
	else
		t->storage->data = realloc(t->storage->data, sizeof(float) * (size_t)stride);
}

void THFloatTensor_resize4d(THFloatTensor *t, long size0, long size1, long size2, long size3)
{
	long s[4] = { size0, size1, size2, size3 };
	THFloatTensor_resize(t, s, 4);
}

void THFloatTensor_resize3d(THFloatTensor *t, long size0, long size1, long size2)
{
	long s[3] = { size0, size1, size2 };
	THFloatTensor_resize(t, s, 3);
}

void THFloatTensor_resize2d(THFloatTensor *t, long size0, long size1)
{
	long s[2] = { size0, size1 };
	THFloatTensor_resize(t, s, 2);
}

void THFloatTensor_resize1d(THFloatTensor *t, long size0)
{
	THFloatTensor_resize(t, &size0, 1);
}

/* tdst becomes another view of tsrc's storage (thbasic.c:282-290). */
void THFloatTensor_set(THFloatTensor *tdst, THFloatTensor *tsrc)
{
	if (tsrc == tdst)
		return;
	if (tsrc->storage)
		__sync_add_and_fetch(&tsrc->storage->nref, 1);
	if (tdst->storage)
		thhip_storage_release(tdst->storage);
	*tdst = *tsrc;
}

THFloatTensor *THFloatTensor_newWithTensor(THFloatTensor *tensor)
{
	THFloatTensor *t = THFloatTensor_new();
	THFloatTensor_set(t, tensor);
	return t;
}

THFloatTensor *THFloatTensor_newWithStorage1d(THFloatStorage *storage, long storageOffset, long size0, long stride0)
{
	THFloatTensor *t = THFloatTensor_new();
	t->nDimension = 1;
	t->size[0] = size0;
	t->stride[0] = stride0 == -1 ? 1 : stride0;
	t->storage = storage;
	t->storageOffset = storageOffset;
	__sync_add_and_fetch(&storage->nref, 1);
	return t;
}

THFloatTensor *THFloatTensor_newWithStorage2d(THFloatStorage *storage, long storageOffset, long size0, long stride0,
	long size1, long stride1)
{
	THFloatTensor *t = THFloatTensor_new();
	t->nDimension = 2;
	t->size[0] = size0;
	t->size[1] = size1;
	t->stride[0] = stride0 == -1 ? size1 : stride0;
	t->stride[1] = stride1 == -1 ? 1 : stride1;
	t->storage = storage;
	t->storageOffset = storageOffset;
	__sync_add_and_fetch(&storage->nref, 1);
	return t;
}
