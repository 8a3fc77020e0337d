/*
 * Command line driver for the MI355X engine, the counterpart of the
 * reference's thnets-test.c:1-207: load a Torch7 model directory, move it to
 * the GPU, run an input through it, print the result and the time per run.
 *
 *   thnets-hip-test -m <model dir> -i <input.t7 | ppm image | random>
 *        [-a <8: fp32 (default), 9: fp16, 10: bf16, 11: uint8>] [-R <uint8 range, default 4>]
 *        [-r runs] [-b nbatch] [-p] [-L max printed] [-l last layer] [-s side] [-P] [-d level]
 *
 * Algorithms 0-7 of the reference (its CPU, cuDNN, OpenCL and 8-bit CPU
 * engines, thnets-test.c:93-95) do not exist in this library; the numbering
 * continues after them.  Inputs: a 3-D (planes x height x width) Float or
 * Double tensor saved with torch.save goes through THProcessFloat, replicated
 * -b times; a binary PPM (P6, 8 bit) goes through THProcessImages the way the
 * reference sends JPEG / PNG files (no image codec is linked here); `random`
 * is a seeded 3 x 224 x 224 tensor of uniform [0, 1) values.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/time.h>
#include "thnets_hip.h"

static double seconds(void)
{
	struct timeval tv;
	gettimeofday(&tv, 0);
	return tv.tv_sec + tv.tv_usec * 1e-6;
}

static unsigned char *load_ppm(const char *path, int *width, int *height)
{
	FILE *fp = fopen(path, "rb");
	if (!fp)
		return 0;
	int maxval = 0, c;
	char magic[3] = { 0 };
	if (fscanf(fp, "%2s", magic) != 1 || strcmp(magic, "P6"))
		goto bad;
	int vals[3], n = 0;
	while (n < 3) {		/* width, height, maxval with # comments between them */
		c = fgetc(fp);
		if (c == '#') {
			while ((c = fgetc(fp)) != '\n' && c != EOF)
				;
		} else if (c >= '0' && c <= '9') {
			ungetc(c, fp);
			if (fscanf(fp, "%d", &vals[n++]) != 1)
				goto bad;
		} else if (c == EOF)
			goto bad;
	}
	fgetc(fp);		/* the single whitespace after maxval */
	*width = vals[0];
	*height = vals[1];
	maxval = vals[2];
	if (maxval != 255 || *width < 1 || *height < 1 || (long)*width * *height > (1L << 28))
		goto bad;
	unsigned char *bitmap = malloc((size_t)*width * *height * 3);
	if (fread(bitmap, 3, (size_t)*width * *height, fp) != (size_t)*width * *height) {
		free(bitmap);
		goto bad;
	}
	fclose(fp);
	return bitmap;
bad:
	fclose(fp);
	return 0;
}

static THFloatTensor *random_input(void)
{
	THFloatTensor *t = THFloatTensor_new();
	THFloatTensor_resize3d(t, 3, 224, 224);
	float *d = THFloatTensor_data(t);
	unsigned long long s = 88172645463325252ull;	/* xorshift64 */
	for (long i = 0; i < 3L * 224 * 224; i++) {
		s ^= s << 13;
		s ^= s >> 7;
		s ^= s << 17;
		d[i] = (float)((s >> 40) * (1.0 / 16777216.0));
	}
	return t;
}

int main(int argc, char **argv)
{
	int runs = 1, print = 0, alg = 8, nbatch = 1, lastlayer = 0x7fffffff, maxoutput = 0x7fffffff, side = 0;
	float range = 4;
	const char *modelsdir = 0, *inputfile = 0;
	for (int i = 1; i < argc; i++) {
		if (argv[i][0] != '-')
			continue;
		const char *arg = i + 1 < argc ? argv[i + 1] : 0;
		switch (argv[i][1]) {
		case 'm': if (arg) modelsdir = argv[++i]; break;
		case 'i': if (arg) inputfile = argv[++i]; break;
		case 'a': if (arg) alg = atoi(argv[++i]); break;
		case 'R': if (arg) range = (float)atof(argv[++i]); break;
		case 'r': if (arg) runs = atoi(argv[++i]); break;
		case 'd': if (arg) th_debug = atoi(argv[++i]); break;
		case 'l': if (arg) lastlayer = atoi(argv[++i]); break;
		case 'L': if (arg) maxoutput = atoi(argv[++i]); break;
		case 's': if (arg) side = atoi(argv[++i]); break;
		case 'b':
			if (arg) {
				nbatch = atoi(argv[++i]);
				if (nbatch > 256 || nbatch < 1)
					nbatch = 256;
			}
			break;
		case 'p': print = 1; break;
		case 'P': th_profile = 1; break;
		case 'M': th_minmax = 1; break;
		}
	}
	if (!modelsdir || !inputfile || alg < 8 || alg > 11 || runs < 1) {
		fprintf(stderr, "Syntax: thnets-hip-test -m <models directory> -i <input.t7 | image.ppm | random>\n");
		fprintf(stderr, "             [-r <number of runs>] [-p(rint results)] [-P(rofile)] [-M(inmax of every layer)]\n");
		fprintf(stderr, "             [-a <alg=8:HIP fp32 (default), 9:HIP fp16, 10:HIP bf16, 11:HIP 8bit>]\n");
		fprintf(stderr, "             [-R <range of the 8 bit activations, default 4>]\n");
		fprintf(stderr, "             [-b <nbatch>] [-d <debuglevel=0 (default),1 or 2>]\n");
		fprintf(stderr, "             [-l <limit last processed layer to this>]\n");
		fprintf(stderr, "             [-L <limit printout to max L numbers>]\n");
		fprintf(stderr, "             [-s <side> (make network spatial)]\n");
		return -1;
	}
	THInit();
	THNETWORK *net = THLoadNetwork(modelsdir);
	if (!net) {
		printf("The network could not be loaded: %d\n", THLastError());
		return 0;
	}
	if (net->net->nelem > lastlayer)
		net->net->nelem = lastlayer;
	if (side)
		THMakeSpatial(net, side);
	if (alg == 9 || alg == 10)
		THHipHalfFloat(alg == 9 ? 1 : 2);
	THNETWORK *dev = alg == 11 ? THCreateHipLowpNetwork(net, range) : THCreateHipNetwork(net);
	THFreeNetwork(net);
	net = dev;

	float *result = 0;
	int n = 0, outwidth = 0, outheight = 0, width, height;
	double t = 0;
	const size_t len = strlen(inputfile);
	unsigned char *bitmap = 0;
	if (len > 4 && !strcmp(inputfile + len - 4, ".ppm") && (bitmap = load_ppm(inputfile, &width, &height))) {
		unsigned char *bitmaps[256];
		for (int i = 0; i < nbatch; i++)
			bitmaps[i] = bitmap;
		/* the first run allocates the module outputs: not timed (thnets-test.c:161-162) */
		THProcessImages(net, bitmaps, nbatch, width, height, 3 * width, &result, &outwidth, &outheight, 0);
		t = seconds();
		for (int i = 0; i < runs; i++)
			n = THProcessImages(net, bitmaps, nbatch, width, height, 3 * width, &result, &outwidth, &outheight, 0);
		t = (seconds() - t) / runs;
		free(bitmap);
	} else {
		THFloatTensor *in = !strcmp(inputfile, "random") ? random_input() : THLoadTensor(inputfile);
		if (!in || in->nDimension != 3) {
			printf("Error loading %s\n", inputfile);
			THFreeNetwork(net);
			return 0;
		}
		const long one = THFloatTensor_nElement(in);
		float *batch = malloc(sizeof(float) * one * nbatch), *work = malloc(sizeof(float) * one * nbatch);
		for (int b = 0; b < nbatch; b++)
			memcpy(batch + b * one, THFloatTensor_data(in), sizeof(float) * one);
		/* THProcessFloat normalises its argument in place: every run gets a fresh copy */
		memcpy(work, batch, sizeof(float) * one * nbatch);
		THProcessFloat(net, work, nbatch, (int)in->size[2], (int)in->size[1], (int)in->size[0], &result, &outwidth, &outheight);
		for (int i = 0; i < runs; i++) {
			memcpy(work, batch, sizeof(float) * one * nbatch);
			const double t0 = seconds();
			n = THProcessFloat(net, work, nbatch, (int)in->size[2], (int)in->size[1], (int)in->size[0], &result, &outwidth,
				&outheight);
			t += seconds() - t0;
		}
		t /= runs;
		free(batch);
		free(work);
		THFloatTensor_free(in);
	}
	if (print) {
		if (n > maxoutput)
			n = maxoutput;
		for (int i = 0; i < n; i++)
			printf("(%d,%d,%d): %f\n", i / (outwidth * outheight), i % (outwidth * outheight) / outwidth, i % outwidth, result[i]);
	}
	printf("1 run processing time: %lf\n", t);
	THFreeNetwork(net);
	return 0;
}
