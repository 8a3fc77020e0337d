/*
 * Torch7 model files for the MI355X engine: a reader for the binary
 * serialisation (`torch.save(path, obj)`, what thload.c:15-426 of the reference
 * reads) and THLoadNetwork (thapi.c:244-333), which turns `<dir>/model.net` and
 * `<dir>/stat.t7` into the host-side `struct network` that THCreateHipNetwork /
 * THCreateHipLowpNetwork upload.  Host code only: nothing here touches the GPU,
 * and nothing here can run a network (this library has no CPU path).
 *
 * File format (all little endian, "long" 8 or 4 bytes depending on the machine
 * that wrote the file):
 *   object  := int32 tag, then by tag
 *     0 nil | 1 number: double | 2 string: int32 n, n bytes | 5 boolean: int32
 *     3 table: int32 index; if the index is new: int32 count, count x (key object, value object)
 *     4 torch: int32 index; if new: string version ("V 1"), string class, payload
 *         torch.XTensor : int32 ndim, long size[ndim], long stride[ndim], long offset (1-based), storage object
 *         torch.XStorage: long n, n raw elements
 *         nn.*          : a table object (the module's fields)
 *     7, 8 function: int32 index, int32 n, n bytes of bytecode, an upvalue object (skipped)
 *   An index seen before names the object already read (shared storages,
 *   shared modules).
 *
 * The document is kept as a tree of t7value; tensors of the network are views
 * into the document's storages, so the document lives as long as the network
 * (it hangs off THNETWORK.netobj and is released by THFreeNetwork).
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "th_engine.h"

enum t7kind { T7_NIL, T7_NUMBER, T7_STRING, T7_BOOLEAN, T7_TABLE, T7_TENSOR, T7_STORAGE, T7_OBJECT, T7_FUNCTION };
enum t7scalar { T7S_BYTE, T7S_CHAR, T7S_SHORT, T7S_INT, T7S_LONG, T7S_FLOAT, T7S_DOUBLE };

#define T7_MAXDIM 8

struct t7value {
	int kind;
	double number;			/* T7_NUMBER, T7_BOOLEAN (0 / 1) */
	char *string;			/* T7_STRING; T7_OBJECT: class name ("nn.Linear") */
	/* T7_TABLE, T7_OBJECT: the fields */
	int nfields;
	struct t7value **keys, **vals;
	/* T7_TENSOR */
	int scalar, ndim;
	long size[T7_MAXDIM], stride[T7_MAXDIM], offset;	/* offset 0-based */
	struct t7value *storage;
	/* T7_STORAGE */
	long nelem;
	void *data;			/* raw elements as stored */
	float *as_float;		/* the same as fp32 (data itself for Float storages) */
	struct t7value *next;		/* every value of a document, for release */
};

struct t7doc {
	struct t7value *all, *root;
	struct t7value **memo;		/* index -> object */
	int nmemo;
	int longsize;
	FILE *fp;
	long filesize;
	int err;
};

static struct t7value *t7_new(struct t7doc *d, int kind)
{
	struct t7value *v = calloc(1, sizeof(*v));
	if (!v)
		THError("out of memory reading a Torch7 file");
	v->kind = kind;
	v->next = d->all;
	d->all = v;
	return v;
}

static void t7_release(struct t7doc *d)
{
	if (!d)
		return;
	for (struct t7value *v = d->all; v;) {
		struct t7value *n = v->next;
		free(v->string);
		free(v->keys);
		free(v->vals);
		if (v->as_float != (float *)v->data)
			free(v->as_float);
		free(v->data);
		free(v);
		v = n;
	}
	free(d->memo);
	free(d);
}

static int t7_fail(struct t7doc *d, int err)
{
	if (!d->err)
		d->err = err;
	return err;
}

static int rd(struct t7doc *d, void *dst, size_t n)
{
	if (d->err)
		return d->err;
	if (fread(dst, 1, n, d->fp) != n)
		return t7_fail(d, ERR_READFILE);
	return 0;
}

static int rd_int(struct t7doc *d)
{
	int32_t v = 0;
	rd(d, &v, 4);
	return v;
}

static long rd_long(struct t7doc *d)
{
	if (d->longsize == 8) {
		int64_t v = 0;
		rd(d, &v, 8);
		return (long)v;
	}
	int32_t v = 0;
	rd(d, &v, 4);
	return v;
}

static char *rd_string(struct t7doc *d)
{
	const int n = rd_int(d);
	if (d->err)
		return 0;
	if (n < 0 || n > (1 << 28)) {
		t7_fail(d, ERR_CORRUPTED);
		return 0;
	}
	char *s = malloc((size_t)n + 1);
	if (!s)
		THError("out of memory reading a Torch7 file");
	s[n] = 0;
	if (rd(d, s, n)) {
		free(s);
		return 0;
	}
	return s;
}

static void memo_put(struct t7doc *d, int idx, struct t7value *v)
{
	if (idx < 0 || idx > (1 << 26)) {
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	if (idx >= d->nmemo) {
		int n = d->nmemo ? d->nmemo : 256;
		while (n <= idx)
			n *= 2;
		d->memo = realloc(d->memo, n * sizeof(*d->memo));
		memset(d->memo + d->nmemo, 0, (n - d->nmemo) * sizeof(*d->memo));
		d->nmemo = n;
	}
	d->memo[idx] = v;
}

static struct t7value *memo_get(struct t7doc *d, int idx)
{
	return idx >= 0 && idx < d->nmemo ? d->memo[idx] : 0;
}

static struct t7value *rd_object(struct t7doc *d, int depth);

static void rd_fields(struct t7doc *d, struct t7value *t, int depth)
{
	const int n = rd_int(d);
	if (d->err)
		return;
	if (n < 0 || n > (1 << 24)) {
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	t->keys = calloc(n ? n : 1, sizeof(*t->keys));
	t->vals = calloc(n ? n : 1, sizeof(*t->vals));
	for (int i = 0; i < n && !d->err; i++) {
		t->keys[i] = rd_object(d, depth + 1);
		t->vals[i] = rd_object(d, depth + 1);
		t->nfields = i + 1;
	}
}

static int scalar_of(const char *name, int *size)
{
	static const struct { const char *name; int scalar, size; } types[] = {
		{ "Byte", T7S_BYTE, 1 }, { "Char", T7S_CHAR, 1 }, { "Short", T7S_SHORT, 2 }, { "Int", T7S_INT, 4 },
		{ "Long", T7S_LONG, 0 }, { "Float", T7S_FLOAT, 4 }, { "Cuda", T7S_FLOAT, 4 }, { "Double", T7S_DOUBLE, 8 },
	};
	for (unsigned i = 0; i < sizeof(types) / sizeof(types[0]); i++)
		if (!strcmp(name, types[i].name)) {
			*size = types[i].size;
			return types[i].scalar;
		}
	return -1;
}

/* "torch.FloatTensor" -> "Float" when the class ends in `suffix` */
static int class_scalar(const char *cls, const char *suffix, int *esize)
{
	const size_t n = strlen(cls), m = strlen(suffix);
	if (n <= 6 + m || memcmp(cls, "torch.", 6) || strcmp(cls + n - m, suffix))
		return -1;
	char name[32];
	if (n - 6 - m >= sizeof(name))
		return -1;
	memcpy(name, cls + 6, n - 6 - m);
	name[n - 6 - m] = 0;
	return scalar_of(name, esize);
}

static void rd_storage(struct t7doc *d, struct t7value *v, int scalar, int esize)
{
	v->kind = T7_STORAGE;
	v->scalar = scalar;
	v->nelem = rd_long(d);
	if (d->err)
		return;
	if (scalar == T7S_LONG)
		esize = d->longsize;
	if (v->nelem < 0 || v->nelem > d->filesize / esize) {	/* also what a wrong long size trips over */
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	v->data = malloc(v->nelem ? (size_t)v->nelem * esize : 1);
	if (!v->data)
		THError("out of memory reading a Torch7 storage of %ld elements", v->nelem);
	if (rd(d, v->data, (size_t)v->nelem * esize))
		return;
	if (scalar == T7S_FLOAT)
		v->as_float = v->data;
	else if (scalar == T7S_DOUBLE) {
		v->as_float = malloc(v->nelem ? sizeof(float) * v->nelem : 1);
		for (long i = 0; i < v->nelem; i++)
			v->as_float[i] = (float)((double *)v->data)[i];
	}
}

static void rd_tensor(struct t7doc *d, struct t7value *v, int scalar, int depth)
{
	v->kind = T7_TENSOR;
	v->scalar = scalar;
	v->ndim = rd_int(d);
	if (d->err)
		return;
	if (v->ndim < 0 || v->ndim > T7_MAXDIM) {
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	for (int i = 0; i < v->ndim; i++)
		v->size[i] = rd_long(d);
	for (int i = 0; i < v->ndim; i++)
		v->stride[i] = rd_long(d);
	v->offset = rd_long(d) - 1;
	struct t7value *st = rd_object(d, depth + 1);
	if (d->err)
		return;
	if (st->kind == T7_NIL)
		return;
	if (st->kind != T7_STORAGE || st->scalar != scalar) {
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	/* every element the sizes and strides reach lies inside the storage */
	long last = v->offset;
	int empty = v->ndim == 0;
	for (int i = 0; i < v->ndim; i++) {
		if (v->size[i] < 0 || v->stride[i] < 0) {
			t7_fail(d, ERR_CORRUPTED);
			return;
		}
		long span;
		if (v->size[i] == 0)
			empty = 1;
		else if (__builtin_mul_overflow(v->size[i] - 1, v->stride[i], &span) || __builtin_add_overflow(last, span, &last)) {
			t7_fail(d, ERR_CORRUPTED);	/* sizes and strides straight from the file: the sum must not wrap */
			return;
		}
	}
	if (!empty && (v->offset < 0 || last >= st->nelem)) {
		t7_fail(d, ERR_CORRUPTED);
		return;
	}
	v->storage = st;
}

static struct t7value *rd_torch(struct t7doc *d, int depth)
{
	const int idx = rd_int(d);
	if (d->err)
		return t7_new(d, T7_NIL);
	struct t7value *seen = memo_get(d, idx);
	if (seen)
		return seen;
	struct t7value *v = t7_new(d, T7_OBJECT);
	memo_put(d, idx, v);
	char *version = rd_string(d);
	if (d->err)
		return v;
	char *cls;
	if (!strncmp(version, "V ", 2))
		cls = rd_string(d);
	else {		/* files older than the version tag start with the class */
		cls = version;
		version = 0;
	}
	free(version);
	if (d->err)
		return v;
	v->string = cls;
	int esize = 0, scalar;
	if ((scalar = class_scalar(cls, "Tensor", &esize)) >= 0)
		rd_tensor(d, v, scalar, depth);
	else if ((scalar = class_scalar(cls, "Storage", &esize)) >= 0)
		rd_storage(d, v, scalar, esize);
	else if (!strncmp(cls, "nn.", 3) || !strncmp(cls, "cudnn.", 6)) {
		struct t7value *t = rd_object(d, depth + 1);
		if (d->err)
			return v;
		if (t->kind != T7_TABLE) {
			t7_fail(d, ERR_CORRUPTED);
			return v;
		}
		/* the object takes over the table's fields */
		v->nfields = t->nfields;
		v->keys = t->keys;
		v->vals = t->vals;
		t->nfields = 0;
		t->keys = t->vals = 0;
	} else
		t7_fail(d, ERR_NOTIMPLEMENTED);
	return v;
}

static struct t7value *rd_object(struct t7doc *d, int depth)
{
	if (depth > 200) {
		t7_fail(d, ERR_CORRUPTED);
		return t7_new(d, T7_NIL);
	}
	const int tag = rd_int(d);
	if (d->err)
		return t7_new(d, T7_NIL);
	struct t7value *v;
	switch (tag) {
	case 0:
		return t7_new(d, T7_NIL);
	case 1:
		v = t7_new(d, T7_NUMBER);
		rd(d, &v->number, 8);
		return v;
	case 2:
		v = t7_new(d, T7_STRING);
		v->string = rd_string(d);
		return v;
	case 5:
		v = t7_new(d, T7_BOOLEAN);
		v->number = rd_int(d) != 0;
		return v;
	case 3: {
		const int idx = rd_int(d);
		if (d->err)
			return t7_new(d, T7_NIL);
		struct t7value *seen = memo_get(d, idx);
		if (seen)
			return seen;
		v = t7_new(d, T7_TABLE);
		memo_put(d, idx, v);
		rd_fields(d, v, depth);
		return v;
	}
	case 4:
		return rd_torch(d, depth);
	case 7:
	case 8: {
		/* a Lua function: bytecode, then its upvalues; kept as a placeholder */
		const int idx = rd_int(d);
		if (d->err)
			return t7_new(d, T7_NIL);
		struct t7value *seen = memo_get(d, idx);
		if (seen)
			return seen;
		v = t7_new(d, T7_FUNCTION);
		memo_put(d, idx, v);
		const int n = rd_int(d);
		if (d->err)
			return v;
		if (n < 0 || fseek(d->fp, n, SEEK_CUR)) {
			t7_fail(d, ERR_READFILE);
			return v;
		}
		rd_object(d, depth + 1);
		return v;
	}
	case 6:
		t7_fail(d, ERR_NOTIMPLEMENTED);
		return t7_new(d, T7_NIL);
	default:
		t7_fail(d, ERR_CORRUPTED);
		return t7_new(d, T7_NIL);
	}
}

/* Reads one file; *err is 0 or one of the ERR_ codes.  A file written with the
 * other long size fails as corrupted (counts and sizes come out absurd), so the
 * caller tries 8 bytes first and then 4, as thapi.c:277-279 does. */
static struct t7doc *t7_read(const char *path, int longsize, int *err)
{
	FILE *fp = fopen(path, "rb");
	if (!fp) {
		*err = ERR_OPENFILE;
		return 0;
	}
	struct t7doc *d = calloc(1, sizeof(*d));
	d->fp = fp;
	d->longsize = longsize;
	fseek(fp, 0, SEEK_END);
	d->filesize = ftell(fp);
	fseek(fp, 0, SEEK_SET);
	d->root = rd_object(d, 0);
	fclose(fp);
	d->fp = 0;
	*err = d->err;
	if (d->err) {
		t7_release(d);
		return 0;
	}
	return d;
}

static struct t7doc *t7_read_any(const char *path, int *err)
{
	struct t7doc *d = t7_read(path, 8, err);
	if (!d && (*err == ERR_CORRUPTED || *err == ERR_READFILE)) {
		int err4;
		d = t7_read(path, 4, &err4);
		if (d)
			*err = 0;
	}
	return d;
}

/* ---- field access ---- */

static struct t7value *field(const struct t7value *t, const char *name)
{
	for (int i = 0; i < t->nfields; i++)
		if (t->keys[i]->kind == T7_STRING && t->keys[i]->string && !strcmp(t->keys[i]->string, name))
			return t->vals[i];
	return 0;
}

/* thload.c:631-651: a missing number reads as 0, a missing boolean as -1 */
static double field_number(const struct t7value *t, const char *name)
{
	const struct t7value *v = field(t, name);
	return v && v->kind == T7_NUMBER ? v->number : 0;
}

static int field_boolean(const struct t7value *t, const char *name)
{
	const struct t7value *v = field(t, name);
	return v && v->kind == T7_BOOLEAN ? (int)v->number : -1;
}

/* A view of a document tensor (thload.c:653-673); an absent field gives an
 * empty tensor, as there. */
static THFloatTensor *tensor_of(const struct t7value *v, const char *what)
{
	THFloatTensor *t = THFloatTensor_new();
	if (!v || v->kind != T7_TENSOR)
		return t;
	if (v->ndim > 4)
		THError("%s: %d-dimensional tensor (at most 4 are supported)", what, v->ndim);
	if (v->scalar != T7S_FLOAT && v->scalar != T7S_DOUBLE)
		THError("%s: only Float / Double / Cuda tensors can be loaded", what);
	t->nDimension = v->ndim;
	for (int i = 0; i < v->ndim; i++) {
		t->size[i] = v->size[i];
		t->stride[i] = v->stride[i];
	}
	t->storageOffset = v->offset;
	if (v->storage)
		t->storage = THFloatStorage_newwithbuffer(v->storage->as_float);
	return t;
}

static THFloatTensor *field_tensor(const struct t7value *t, const char *name, const char *cls)
{
	char what[96];
	snprintf(what, sizeof(what), "%s.%s", cls, name);
	return tensor_of(field(t, name), what);
}

/* ---- nn objects -> struct module ---- */

static struct network *network_of(const struct t7value *container);

static void free_conv(struct module *m)
{
	THFloatTensor_free(m->SpatialConvolution.bias);
	THFloatTensor_free(m->SpatialConvolution.weight);
	THFloatTensor_free(m->SpatialConvolution.finput);
}

static void free_linear(struct module *m)
{
	THFloatTensor_free(m->Linear.bias);
	THFloatTensor_free(m->Linear.weight);
	THFloatTensor_free(m->Linear.addBuffer);
}

static void free_bn(struct module *m)
{
	THFloatTensor_free(m->SpatialBatchNormalization.running_mean);
	THFloatTensor_free(m->SpatialBatchNormalization.running_var);
	THFloatTensor_free(m->SpatialBatchNormalization.weight);
	THFloatTensor_free(m->SpatialBatchNormalization.bias);
}

static void free_fullconv(struct module *m)
{
	THFloatTensor_free(m->SpatialFullConvolution.bias);
	THFloatTensor_free(m->SpatialFullConvolution.weight);
	THFloatTensor_free(m->SpatialFullConvolution.ones);
	THFloatTensor_free(m->SpatialFullConvolution.columns);
}

static void free_host_network(struct network *net);

static void free_container(struct module *m)
{
	if (m->Sequential.net)
		free_host_network(m->Sequential.net);
}

/* modules/SpatialConvolution.c:11-35 */
static void load_conv(struct module *m, const struct t7value *o)
{
	struct SpatialConvolution *c = &m->SpatialConvolution;
	m->type = MT_SpatialConvolutionVirtMM;	/* what THUseSpatialConvolutionMM(net, 2) leaves, thapi.c:331 */
	m->nnfree = free_conv;
	c->padW = (int)field_number(o, "padW");
	c->padH = (int)field_number(o, "padH");
	if (!c->padW && !c->padH)
		c->padW = c->padH = (int)field_number(o, "padding");
	c->dW = (int)field_number(o, "dW");
	c->dH = (int)field_number(o, "dH");
	c->kW = (int)field_number(o, "kW");
	c->kH = (int)field_number(o, "kH");
	c->nInputPlane = (int)field_number(o, "nInputPlane");
	c->nOutputPlane = (int)field_number(o, "nOutputPlane");
	c->bias = field_tensor(o, "bias", o->string);
	c->weight = field_tensor(o, "weight", o->string);
	c->finput = THFloatTensor_new();
	THFloatTensor *w = c->weight;
	if (!w->storage || (w->nDimension != 2 && w->nDimension != 4))
		THError("%s: weight must be a 2-D or 4-D tensor", o->string);
	if (w->nDimension == 4) {	/* [Co][Ci][kH][kW] is read as [Co][Ci*kH*kW]: only when it lies that way */
		if (w->stride[3] != 1 || w->stride[2] != w->size[3] || w->stride[1] != w->size[2] * w->size[3] ||
		    w->stride[0] != w->size[1] * w->size[2] * w->size[3])
			THError("%s: 4-D weight is not contiguous", o->string);
		w->size[1] *= w->size[2] * w->size[3];
		w->stride[1] = 1;
		w->nDimension = 2;
	}
	if (c->dW < 1 || c->dH < 1 || c->kW < 1 || c->kH < 1 || w->size[0] != c->nOutputPlane ||
	    w->size[1] != (long)c->nInputPlane * c->kH * c->kW || w->stride[1] != 1 || w->stride[0] != w->size[1])
		THError("%s: weight %ldx%ld does not fit %d -> %d planes, kernel %dx%d", o->string, w->size[0], w->size[1],
			c->nInputPlane, c->nOutputPlane, c->kH, c->kW);
}

static void load_pool(struct module *m, const struct t7value *o, int average)
{
	/* the two parameter blocks start with the same seven ints */
	struct SpatialMaxPooling *p = &m->SpatialMaxPooling;
	m->type = average ? MT_SpatialAveragePooling : MT_SpatialMaxPooling;
	p->padW = (int)field_number(o, "padW");
	p->padH = (int)field_number(o, "padH");
	p->dW = (int)field_number(o, "dW");
	p->dH = (int)field_number(o, "dH");
	p->kW = (int)field_number(o, "kW");
	p->kH = (int)field_number(o, "kH");
	/* Torch writes ceil_mode as a boolean; the reference reads a number
	 * (SpatialMaxPooling.c:22) and so always gets floor mode.  Both spellings
	 * are honoured here. */
	const struct t7value *cm = field(o, "ceil_mode");
	p->ceil_mode = cm && (cm->kind == T7_NUMBER || cm->kind == T7_BOOLEAN) ? cm->number != 0 : 0;
	if (average) {
		const struct t7value *cp = field(o, "count_include_pad");
		m->SpatialAveragePooling.count_include_pad = cp && (cp->kind == T7_NUMBER || cp->kind == T7_BOOLEAN) ? cp->number != 0 : 0;
	}
}

static void load_module(struct module *m, const struct t7value *o)
{
	const char *cls = o->string;
	if (!strcmp(cls, "nn.SpatialConvolutionMM") || !strcmp(cls, "nn.SpatialConvolution") || !strcmp(cls, "cudnn.SpatialConvolution"))
		load_conv(m, o);
	else if (!strcmp(cls, "nn.SpatialMaxPooling") || !strcmp(cls, "cudnn.SpatialMaxPooling"))
		load_pool(m, o, 0);
	else if (!strcmp(cls, "nn.SpatialAveragePooling") || !strcmp(cls, "cudnn.SpatialAveragePooling"))
		load_pool(m, o, 1);
	else if (!strcmp(cls, "nn.Linear")) {		/* modules/Linear.c:10-22 */
		m->type = MT_Linear;
		m->nnfree = free_linear;
		m->Linear.weight = field_tensor(o, "weight", cls);
		m->Linear.bias = field_tensor(o, "bias", cls);
		m->Linear.addBuffer = THFloatTensor_new();
		THFloatTensor *w = m->Linear.weight;
		if (!w->storage || w->nDimension != 2 || w->stride[1] != 1 || w->stride[0] != w->size[1])
			THError("nn.Linear: weight must be a contiguous 2-D tensor");
	} else if (!strcmp(cls, "nn.Threshold") || !strcmp(cls, "nn.ReLU") || !strcmp(cls, "cudnn.ReLU")) {
		m->type = MT_Threshold;			/* modules/Threshold.c:3-13 */
		m->Threshold.threshold = (float)field_number(o, "threshold");
		m->Threshold.val = (float)field_number(o, "val");
		m->Threshold.alpha = 0;
		m->Threshold.inplace = field_boolean(o, "inplace");
	} else if (!strcmp(cls, "nn.SoftMax") || !strcmp(cls, "cudnn.SoftMax"))
		m->type = MT_SoftMax;
	else if (!strcmp(cls, "nn.View")) {
		m->type = MT_View;
		m->View.numElements = (int)field_number(o, "numElements");
	} else if (!strcmp(cls, "nn.Reshape")) {
		/* a flattening Reshape is a View (modules/Reshape.c:7-20 keeps the
		 * size list; only the one-dimensional case is served here) */
		const struct t7value *sz = field(o, "size");
		if (!sz || sz->kind != T7_STORAGE || sz->nelem != 1)
			THError("nn.Reshape: only a reshape to one dimension is supported");
		m->type = MT_View;
		m->View.numElements = (int)field_number(o, "nelement");
	} else if (!strcmp(cls, "nn.Dropout") || !strcmp(cls, "nn.SpatialDropout") || !strcmp(cls, "nn.Identity")) {
		m->type = MT_Dropout;			/* modules/Dropout.c:3-13: identity at inference */
		m->Dropout.inplace = field_boolean(o, "inplace");
		m->Dropout.v2 = field_boolean(o, "v2");
		m->Dropout.p = (float)field_number(o, "p");
	} else if (!strcmp(cls, "nn.SpatialBatchNormalization") || !strcmp(cls, "cudnn.SpatialBatchNormalization")) {
		struct SpatialBatchNormalization *b = &m->SpatialBatchNormalization;
		m->type = MT_SpatialBatchNormalization;	/* modules/SpatialBatchNormalization.c:12-25 */
		m->nnfree = free_bn;
		b->running_mean = field_tensor(o, "running_mean", cls);
		b->running_var = field_tensor(o, "running_var", cls);
		b->weight = field_tensor(o, "weight", cls);
		b->bias = field_tensor(o, "bias", cls);
		b->eps = field_number(o, "eps");
		if (!b->running_mean->storage || !b->running_var->storage)
			THError("nn.SpatialBatchNormalization: running_mean / running_var are missing");
	} else if (!strcmp(cls, "nn.Sequential") || !strcmp(cls, "nn.ConcatTable")) {
		m->type = cls[3] == 'S' ? MT_Sequential : MT_ConcatTable;
		m->nnfree = free_container;
		m->Sequential.net = network_of(o);
		if (!m->Sequential.net)
			THError("%s without a module list", cls);
	} else if (!strcmp(cls, "nn.SpatialFullConvolution")) {
		struct SpatialFullConvolution *c = &m->SpatialFullConvolution;
		m->type = MT_SpatialFullConvolution;	/* modules/SpatialFullConvolution.c:12-35 */
		m->nnfree = free_fullconv;
		c->padW = (int)field_number(o, "padW");
		c->padH = (int)field_number(o, "padH");
		c->adjW = (int)field_number(o, "adjW");
		c->adjH = (int)field_number(o, "adjH");
		c->dW = (int)field_number(o, "dW");
		c->dH = (int)field_number(o, "dH");
		c->kW = (int)field_number(o, "kW");
		c->kH = (int)field_number(o, "kH");
		c->nInputPlane = (int)field_number(o, "nInputPlane");
		c->nOutputPlane = (int)field_number(o, "nOutputPlane");
		c->bias = field_tensor(o, "bias", cls);
		c->weight = field_tensor(o, "weight", cls);
		c->columns = THFloatTensor_new();
		c->ones = THFloatTensor_new();
		if (!c->weight->storage || c->weight->nDimension != 4)
			THError("nn.SpatialFullConvolution: weight must be a 4-D tensor");
	} else if (!strcmp(cls, "nn.SpatialMaxUnpooling")) {
		/* modules/SpatialMaxUnpooling.c:4-12: the pooling module is named by its
		 * loader object, which SpatialMaxPooling modules carry in `nnmodule` */
		const struct t7value *pool = field(o, "pooling");
		if (!pool || pool->kind != T7_OBJECT)
			THError("nn.SpatialMaxUnpooling without its pooling module");
		m->type = MT_SpatialMaxUnpooling;
		m->SpatialMaxUnpooling.pooling = (void *)pool;
	} else if (!strcmp(cls, "nn.CAddTable"))
		m->type = MT_CAddTable;
	else if (!strcmp(cls, "nn.CSubTable"))
		m->type = MT_CSubTable;
	else
		THError("Unknown module type %s", cls);		/* thload.c:776 */
}

/* thload.c:744-781.  The `modules` table is an array: keys 1..n. */
static struct network *network_of(const struct t7value *container)
{
	const struct t7value *mods = field(container, "modules");
	if (!mods || mods->kind != T7_TABLE)
		return 0;
	int n = 0;
	for (int i = 0; i < mods->nfields; i++)
		if (mods->keys[i]->kind == T7_NUMBER && mods->vals[i]->kind == T7_OBJECT)
			n++;
	struct network *net = calloc(1, sizeof(*net));
	net->engine = ENGINE_CPU;
	net->nelem = n;
	net->modules = calloc(n ? n : 1, sizeof(*net->modules));
	for (int i = 0; i < mods->nfields; i++) {
		if (mods->keys[i]->kind != T7_NUMBER || mods->vals[i]->kind != T7_OBJECT)
			continue;
		const double key = mods->keys[i]->number;
		const int pos = (int)key - 1;
		if (key != (double)(pos + 1) || pos < 0 || pos >= n || net->modules[pos].net)
			THError("%s: the module list is not an array 1..%d", container->string, n);
		struct module *m = net->modules + pos;
		m->net = net;
		m->output = THFloatTensor_new();
		m->nnmodule = (void *)mods->vals[i];
		load_module(m, mods->vals[i]);
	}
	return net;
}

/* thload.c:783-803 */
static void free_host_network(struct network *net)
{
	for (int i = 0; i < net->nelem; i++) {
		struct module *m = net->modules + i;
		if (m->nnfree)
			m->nnfree(m);
		if (m->output)
			THFloatTensor_free(m->output);
	}
	free(net->modules);
	free(net);
}

static int g_load_error;

int thhip_load_error(void)
{
	return g_load_error;
}

/* thapi.c:244-333 for Torch7 model directories: <path>/model.net holds the
 * nn.Sequential, <path>/stat.t7 (optional) a table {mean = tensor, std = tensor}.
 * Returns 0 and leaves the reason in THLastError() when the files cannot be
 * read; a network this engine cannot represent is fatal, as in the reference. */
THNETWORK *THLoadNetwork(const char *path)
{
	char file[1024];
	g_load_error = 0;
	if (snprintf(file, sizeof(file), "%s/model.net", path) >= (int)sizeof(file)) {
		g_load_error = ERR_OPENFILE;
		return 0;
	}
	struct t7doc *d = t7_read_any(file, &g_load_error);
	if (!d)
		return 0;
	if (d->root->kind != T7_OBJECT || strncmp(d->root->string, "nn.", 3)) {
		g_load_error = ERR_WRONGOBJECT;
		t7_release(d);
		return 0;
	}
	struct network *net = network_of(d->root);
	if (!net) {
		g_load_error = ERR_WRONGOBJECT;
		t7_release(d);
		return 0;
	}
	THNETWORK *n = calloc(1, sizeof(*n));
	n->netobj = d;
	n->net = net;
	for (int i = 0; i < 3; i++) {
		n->mean[i] = 0;
		n->std[i] = 1;
	}
	snprintf(file, sizeof(file), "%s/stat.t7", path);
	int err;
	struct t7doc *s = t7_read_any(file, &err);
	if (s) {
		const struct t7value *mean = field(s->root, "mean"), *std = field(s->root, "std");
		if (s->root->kind != T7_TABLE || s->root->nfields != 2 || !mean || !std || mean->kind != T7_TENSOR ||
		    std->kind != T7_TENSOR || !mean->storage || !std->storage || mean->ndim != 1 || std->ndim != 1 ||
		    mean->size[0] < 3 || std->size[0] < 3 || !mean->storage->as_float || !std->storage->as_float) {
			g_load_error = ERR_WRONGOBJECT;
			t7_release(s);
			free_host_network(net);
			t7_release(d);
			free(n);
			return 0;
		}
		for (int i = 0; i < 3; i++) {
			n->mean[i] = mean->storage->as_float[mean->offset + i * mean->stride[0]];
			n->std[i] = std->storage->as_float[std->offset + i * std->stride[0]];
		}
		t7_release(s);
	}
	return n;
}

/* Releases a network made by THLoadNetwork (the host description and the
 * document its tensors point into). */
void thhip_free_loaded_network(THNETWORK *n)
{
	free_host_network(n->net);
	t7_release(n->netobj);
	if (n->out)
		THFloatTensor_free(n->out);
	free(n);
}

/* A Float / Double tensor saved with torch.save, as a new contiguous host
 * tensor that owns its memory (what thnets-test.c:166-178 does with
 * loadtorch + THFloatTensor_newFromObject for its `-i file.t7` input).
 * Returns 0 with the reason in THLastError(). */
THFloatTensor *THLoadTensor(const char *path)
{
	g_load_error = 0;
	struct t7doc *d = t7_read_any(path, &g_load_error);
	if (!d)
		return 0;
	const struct t7value *v = d->root;
	if (v->kind != T7_TENSOR || !v->storage || !v->storage->as_float || v->ndim < 1 || v->ndim > 4) {
		g_load_error = ERR_WRONGOBJECT;
		t7_release(d);
		return 0;
	}
	THFloatTensor *t = THFloatTensor_new();
	long size[4];
	for (int i = 0; i < v->ndim; i++)
		size[i] = v->size[i];
	THFloatTensor_resize(t, size, v->ndim);
	float *dst = THFloatTensor_data(t);
	long idx[4] = { 0, 0, 0, 0 };
	const long total = THFloatTensor_nElement(t);
	for (long e = 0; e < total; e++) {
		long off = v->offset;
		for (int i = 0; i < v->ndim; i++)
			off += idx[i] * v->stride[i];
		dst[e] = v->storage->as_float[off];
		for (int i = v->ndim - 1; i >= 0; i--) {
			if (++idx[i] < v->size[i])
				break;
			idx[i] = 0;
		}
	}
	t7_release(d);
	return t;
}
