/*
 * Binary data-set readers and the driver around the KFAC trust-region solver: host code that stands
 * either side of the solver in the reference (utilities/dataset.c, drivers/dataset_driver.c,
 * drivers/kfac_trust_region_driver.cu).  Records are transposed into the column-major image layout while
 * they are read, so no second host copy of the set is needed.
 */
#define _GNU_SOURCE
#include <limits.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "fitre_dataset.h"
#include "fitre_shim.h"

#define CIFAR10_RECORD 3073
#define CIFAR100_RECORD 3074
#define TINY_RECORD (64 * 64 * 3 + 1)
#define PATH_BYTES 1024

/* drivers/dataset_driver.c:66,85,104 and drivers/kfac_trust_region_driver.cu:205 */
static const char *kDefaultDatasetFolder[3] = {
	"/scratch/gilbreth/skylasa/datasets/cifar/cifar-10-batches-bin/",
	"/scratch/gilbreth/skylasa/datasets/cifar/cifar-100-binary/",
	"/scratch/gilbreth/skylasa/datasets/tiny-imagenet-200/files/",
};
static const char *kDefaultWeightsFolder = "/scratch/gilbreth/skylasa/weights/";
static char g_datasetFolder[3][PATH_BYTES];
static char g_weightsFolder[PATH_BYTES];

void fitreSetDatasetFolder(int datasetType, const char *dir)
{
	if (datasetType < 1 || datasetType > 3) {
		fprintf(stderr, "fitreSetDatasetFolder: unknown datasetType %d\n", datasetType);
		exit(-1);
	}
	char *slot = g_datasetFolder[datasetType - 1];
	slot[0] = 0;
	if (dir != NULL) snprintf(slot, PATH_BYTES, "%s", dir);
}

void fitreSetWeightsFolder(const char *dir)
{
	g_weightsFolder[0] = 0;
	if (dir != NULL) snprintf(g_weightsFolder, PATH_BYTES, "%s", dir);
}

static const char *dataset_folder(int datasetType)
{
	const char *set = g_datasetFolder[datasetType - 1];
	return set[0] ? set : kDefaultDatasetFolder[datasetType - 1];
}

static const char *weights_folder(void) { return g_weightsFolder[0] ? g_weightsFolder : kDefaultWeightsFolder; }

void convertToColumnMajor(real *src, int rows, int cols, real *tgt)
{
	for (int i = 0; i < rows; i++)
		for (int j = 0; j < cols; j++) tgt[(size_t)j * rows + i] = src[(size_t)i * cols + j];
}

void convertCIFARToColumnMajor(real *src, real *tgt, int datasetSize, int channels, int height, int width)
{
	const size_t cells = (size_t)height * width;
	for (size_t plane = 0; plane < (size_t)datasetSize * channels; plane++) {
		const real *s = src + plane * cells;
		real *t = tgt + plane * cells;
		for (int row = 0; row < height; row++)
			for (int col = 0; col < width; col++) t[(size_t)col * height + row] = s[(size_t)row * width + col];
	}
}

void imageNormalization(real *src, int numImages, int channels, int height, int width, real constant, int datasetType)
{
	static const real mean[3][3] = { { 0.4914, 0.4822, 0.4465 }, { 0.5071, 0.4865, 0.4409 }, { 0.4799, 0.4478, 0.3972 } };
	static const real std[3][3] = { { 0.2470, 0.2435, 0.2616 }, { 0.2673, 0.2564, 0.2762 }, { 0.2769, 0.2690, 0.2820 } };
	if (datasetType < 1 || datasetType > 3) {
		fprintf(stderr, "Unknown DatasetType here... \n\n");
		exit(-1);
	}
	const size_t perChannel = (size_t)height * width * numImages;
	for (int c = 0; c < channels; c++) {
		real *p = src + c * perChannel;
		const real m = mean[datasetType - 1][c % 3], s = std[datasetType - 1][c % 3];
		for (size_t i = 0; i < perChannel; i++) p[i] = (p[i] / constant - m) / s;
	}
}

/* ---- delimited text ---------------------------------------------------------------------------- */

static int count_tokens(const char *line)
{
	int n = 0, inToken = 0;
	for (const char *c = line; *c; c++) {
		const int sep = *c == ',' || *c == ' ' || *c == '\n' || *c == '\r' || *c == '\t';
		if (!sep && !inToken) n++;
		inToken = !sep;
	}
	return n;
}

void readDelimitedMatrix(char *fileName, real **data, int *rows, int *cols)
{
	FILE *f = fopen(fileName, "r");
	fprintf(stderr, "Reading file: %s \n", fileName);
	if (f == NULL) {
		fprintf(stderr, "Error opening the dataset.... !\n");
		exit(-1);
	}
	char *line = NULL;
	size_t cap = 0;
	*rows = *cols = 0;
	int ragged = 0, first = 0;
	while (getline(&line, &cap, f) > 0) { /* first pass: the shape; an empty line ends the matrix */
		const int n = count_tokens(line);
		if (n == 0) break;
		if (*rows == 0) first = n;
		if (n != first) ragged++;
		*cols = n;
		(*rows)++;
	}
	/* an empty line in the middle of a file, or rows of different lengths, give a matrix that is not what the file
	 * holds: say so (the shape is still taken as before: rows up to the empty line, columns of the last row) */
	while (getline(&line, &cap, f) > 0)
		if (count_tokens(line) > 0) {
			fprintf(stderr, "readDelimitedMatrix: %s: stopped at the empty line after row %d, but more rows follow\n", fileName, *rows);
			break;
		}
	if (ragged)
		fprintf(stderr, "readDelimitedMatrix: %s: %d of %d rows do not have the %d values of the first row; missing values read as 0\n",
		        fileName, ragged, *rows, first);
	fprintf(stderr, "Rows : %d, Columns : %d \n", *rows, *cols);
	const size_t total = (size_t)*rows * (size_t)*cols;
	*data = (real *)calloc(total > 0 ? total : 1, sizeof(real));
	if (*data == NULL) {
		fprintf(stderr, "readDelimitedMatrix: no host memory for %d x %d values\n", *rows, *cols);
		exit(-1);
	}
	rewind(f);
	for (int r = 0; r < *rows && getline(&line, &cap, f) > 0; r++) {
		int c = 0;
		for (char *word = strtok(line, ", \n\r\t"); word != NULL && c < *cols; word = strtok(NULL, ", \n\r\t"))
			(*data)[(size_t)r * *cols + c++] = (real)atof(word);
	}
	free(line);
	fclose(f);
	fprintf(stderr, "Done reading: %s \n", fileName);
}

/* ---- record files ---------------------------------------------------------------------------- */

typedef struct record_format {
	size_t recordBytes;
	int labelByte;  /* which byte of the record holds the label that is kept */
	int pixelStart; /* first pixel byte */
	int classes;
} RECORD_FORMAT;

static RECORD_FORMAT record_format(int datasetType)
{
	RECORD_FORMAT f = { 0, 0, 0, 0 };
	switch (datasetType) {
	case 1: f.recordBytes = CIFAR10_RECORD, f.labelByte = 0, f.pixelStart = 1, f.classes = 10; break;
	case 2: f.recordBytes = CIFAR100_RECORD, f.labelByte = 1, f.pixelStart = 2, f.classes = 100; break;
	case 3: f.recordBytes = TINY_RECORD, f.labelByte = 0, f.pixelStart = 1, f.classes = 200; break;
	default:
		fprintf(stderr, "readCIFARDataset: unknown datasetType %d\n", datasetType);
		exit(-1);
	}
	return f;
}

static FILE *open_or_exit(const char *filename)
{
	FILE *f = fopen(filename, "rb");
	if (f == NULL) {
		fprintf(stderr, "Error opening the dataset.... ! (%s)\n", filename);
		exit(-1);
	}
	return f;
}

/* records in the file; a trailing partial record counts (utilities/dataset.c:287-305 reads until fread
 * returns nothing and zero-fills the line buffer before each read) */
static long count_records(const char *filename, size_t recordBytes)
{
	FILE *f = open_or_exit(filename);
	fseek(f, 0, SEEK_END);
	long bytes = ftell(f);
	fclose(f);
	return (bytes + (long)recordBytes - 1) / (long)recordBytes;
}

/* appends the file's records at image index `count`; returns the new count */
static long read_records(const char *filename, RECORD_FORMAT fmt, int channels, int height, int width, real *labels,
                         real *images, long count)
{
	FILE *f = open_or_exit(filename);
	unsigned char *line = (unsigned char *)malloc(fmt.recordBytes);
	const size_t cells = (size_t)height * width, features = cells * channels;
	int minLabel = INT_MAX, maxLabel = 0;
	for (;;) {
		memset(line, 0, fmt.recordBytes);
		if (fread(line, 1, fmt.recordBytes, f) == 0) break;
		const int label = (int)line[fmt.labelByte] + 1;
		if (label < minLabel) minLabel = label;
		if (label > maxLabel) maxLabel = label;
		labels[count] = (real)label;
		real *img = images + (size_t)count * features;
		const unsigned char *px = line + fmt.pixelStart;
		for (int c = 0; c < channels; c++)
			for (int row = 0; row < height; row++)
				for (int col = 0; col < width; col++)
					img[c * cells + (size_t)col * height + row] = (real)px[c * cells + (size_t)row * width + col];
		count++;
	}
	free(line);
	fclose(f);
	fprintf(stderr, "Done with reading %ld points from the input files, Label( %d, %d ) .... \n", count, minLabel, maxLabel);
	return count;
}

void readCIFARDataset(char *dir, char *train, int numFiles, char *test, HOST_DATASET *data, SCRATCH_AREA *s, int raw,
                      int batchSize, int datasetType, int height, int width)
{
	(void)s;
	(void)raw;
	(void)batchSize;
	const RECORD_FORMAT fmt = record_format(datasetType);
	const int channels = 3;
	const size_t features = fmt.recordBytes - (size_t)fmt.pixelStart;
	if ((size_t)channels * height * width != features) {
		fprintf(stderr, "readCIFARDataset: %d x %d x %d images do not fill a record of %zu pixel bytes\n", channels, height,
		        width, features);
		exit(-1);
	}
	char filename[PATH_BYTES];
	const int testFiles = datasetType == 3 ? 2 : 1;

	long trainImages = 0, testImages = 0;
	for (int idx = 1; idx <= numFiles; idx++) {
		snprintf(filename, PATH_BYTES, "%s%s%d.bin", dir, train, idx);
		trainImages += count_records(filename, fmt.recordBytes);
	}
	for (int idx = 1; idx <= testFiles; idx++) {
		if (datasetType == 3)
			snprintf(filename, PATH_BYTES, "%s%s%d.bin", dir, test, idx);
		else
			snprintf(filename, PATH_BYTES, "%s%s", dir, test);
		testImages += count_records(filename, fmt.recordBytes);
	}
	fprintf(stderr, "Train Images: %ld \n", trainImages);

	real *trainSet = (real *)malloc(sizeof(real) * (size_t)(trainImages > 0 ? trainImages : 1) * features);
	real *trainLabels = (real *)malloc(sizeof(real) * (size_t)(trainImages > 0 ? trainImages : 1));
	real *testSet = (real *)malloc(sizeof(real) * (size_t)(testImages > 0 ? testImages : 1) * features);
	real *testLabels = (real *)malloc(sizeof(real) * (size_t)(testImages > 0 ? testImages : 1));
	if (!trainSet || !trainLabels || !testSet || !testLabels) {
		fprintf(stderr, "readCIFARDataset: out of host memory for %ld + %ld images\n", trainImages, testImages);
		exit(-1);
	}

	long count = 0;
	for (int idx = 1; idx <= numFiles; idx++) {
		snprintf(filename, PATH_BYTES, "%s%s%d.bin", dir, train, idx);
		fprintf(stderr, "Reading file : %s \n", filename);
		count = read_records(filename, fmt, channels, height, width, trainLabels, trainSet, count);
	}
	count = 0;
	for (int idx = 1; idx <= testFiles; idx++) {
		if (datasetType == 3)
			snprintf(filename, PATH_BYTES, "%s%s%d.bin", dir, test, idx);
		else
			snprintf(filename, PATH_BYTES, "%s%s", dir, test);
		fprintf(stderr, "Reading file : %s \n", filename);
		count = read_records(filename, fmt, channels, height, width, testLabels, testSet, count);
	}

	data->trainSizeX = data->trainSizeY = (int)trainImages;
	data->testSizeX = data->testSizeY = (int)testImages;
	data->trainSetX = trainSet;
	data->trainSetY = trainLabels;
	data->testSetX = testSet;
	data->testSetY = testLabels;
	data->features = (int)features;
	data->numClasses = fmt.classes;
}

/* ---- device copies ---------------------------------------------------------------------------- */

static void copy_sizes(const HOST_DATASET *s, DEVICE_DATASET *t)
{
	t->trainSizeX = s->trainSizeX;
	t->trainSizeY = s->trainSizeY;
	t->testSizeX = s->testSizeX;
	t->testSizeY = s->testSizeY;
	t->features = s->features;
	t->height = s->height;
	t->width = s->width;
	t->numClasses = s->numClasses;
	fprintf(stderr, "Dataset Report: ...\nTrain Set Size: %d \nFeatures: %d \nnumClasses: %d \n", s->trainSizeX, s->features,
	        s->numClasses);
}

static void upload(real **dev, real *host, size_t reals, int err)
{
	cuda_malloc((void **)dev, (reals > 0 ? reals : 1) * sizeof(real), 0, ERROR_MEM_ALLOC);
	if (reals > 0) copy_host_device(host, *dev, reals * sizeof(real), cudaMemcpyHostToDevice, err);
}

void initialize_device_data(HOST_DATASET *s, DEVICE_DATASET *t)
{
	copy_sizes(s, t);
	upload(&t->trainSetX, s->trainSetX, (size_t)t->trainSizeX * t->features, ERROR_MEMCPY_TRAINSETX);
	upload(&t->trainSetY, s->trainSetY, (size_t)t->trainSizeX, ERROR_MEMCPY_TRAINSETY);
	upload(&t->testSetX, s->testSetX, (size_t)t->testSizeX * t->features, ERROR_MEMCPY_TESTSETX);
	upload(&t->testSetY, s->testSetY, (size_t)t->testSizeX, ERROR_MEMCPY_TESTSETY);
	fprintf(stderr, "Train Set size: %d, %d, %d \nTest Set size: %d, %d, %d \n", t->features, t->trainSizeX, t->numClasses,
	        t->features, t->testSizeX, t->numClasses);
}

void initialize_device_image(HOST_DATASET *s, DEVICE_DATASET *t)
{
	copy_sizes(s, t);
	t->trainSetX = NULL;
	t->trainSetY = NULL;
	upload(&t->testSetX, s->testSetX, (size_t)t->testSizeX * t->features, ERROR_MEMCPY_TESTSETX);
	upload(&t->testSetY, s->testSetY, (size_t)t->testSizeX, ERROR_MEMCPY_TESTSETY);
	fprintf(stderr, "Train Set size (host): %d, %d, %d \nTest Set size: %d, %d, %d \n", t->features, t->trainSizeX,
	        t->numClasses, t->features, t->testSizeX, t->numClasses);
}

void cleanup_dataset(HOST_DATASET *s, DEVICE_DATASET *t)
{
	real **hostArrays[4] = { &s->trainSetX, &s->trainSetY, &s->testSetX, &s->testSetY };
	real **devArrays[4] = { &t->trainSetX, &t->trainSetY, &t->testSetX, &t->testSetY };
	for (int i = 0; i < 4; i++) {
		if (*hostArrays[i]) free(*hostArrays[i]);
		*hostArrays[i] = NULL;
		if (*devArrays[i]) cuda_free(*devArrays[i], ERROR_MEM_CLEANUP);
		*devArrays[i] = NULL;
	}
}

static int get_dataset(int datasetType, DATASET_TYPE tag, int side, char *train, int trainFiles, char *test, int onDevice,
                       CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch)
{
	char dir[PATH_BYTES];
	snprintf(dir, PATH_BYTES, "%s", dataset_folder(datasetType));
	host->height = side;
	host->width = side;
	host->datasetType = device->datasetType = tag;
	readCIFARDataset(dir, train, trainFiles, test, host, scratch, 255, model->batchSize, datasetType, side, side);
	if (onDevice)
		initialize_device_data(host, device);
	else
		initialize_device_image(host, device);
	fprintf(stderr, "Done reading the dataset .... \n");
	return 0;
}

int getCIFAR10(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch)
{
	fprintf(stderr, "Reading CIFAR_10 dataset... \n");
	return get_dataset(1, CIFAR10, 32, "data_batch_", 5, "test_batch.bin", 1, model, host, device, scratch);
}

int getCIFAR100(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch)
{
	fprintf(stderr, "Reading CIFAR_100 dataset... \n");
	return get_dataset(2, CIFAR100, 32, "train_", 1, "test.bin", 1, model, host, device, scratch);
}

int getTinyImageNet(CNN_MODEL *model, HOST_DATASET *host, DEVICE_DATASET *device, SCRATCH_AREA *scratch)
{
	fprintf(stderr, "Reading Tiny ImageNet dataset... \n");
	return get_dataset(3, IMAGENET, 64, "train_", 19, "test_", 0, model, host, device, scratch);
}

void cnnInitializations(CNN_MODEL *model, DEVICE_DATASET *data)
{
	fprintf(stderr, "Weights Size: %d \n", model->pSize);
	cuda_malloc((void **)&data->weights, (size_t)model->pSize * sizeof(real), 0, ERROR_MEM_ALLOC);
}

/* ---- the driver -------------------------------------------------------------------------------- */

void initKFACTrustRegionParams(TRUST_REGION_PARAMS *params, int n)
{
	(void)n;
	params->eta1 = 0.8;
	params->eta2 = 1e-4;
	params->gamma1 = 2;
	params->gamma2 = 1.2;
	params->maxProps = ULONG_MAX;
	params->maxMatVecs = INT_MAX; /* the reference assigns 1e15 to this int, which does not fit */
	params->maxEpochs = 1;
	params->hessianType = TRUE_HESSIAN;
	params->hs = 0;
	params->delta = 1.;
	params->maxDelta = 100;
	params->minDelta = 1e-6;
	params->maxIters = 200;
	params->alpha = 0.01;
	params->lambda = 0;
	params->curIteration = 0;
}

void initKFACInfo(KFAC_CURVATURE_INFO *kfacInfo)
{
	memset(kfacInfo, 0, sizeof(*kfacInfo));
	kfacInfo->stats_decay = 0.8;
	kfacInfo->momentum = 0;
	kfacInfo->regLambda = 1e-3;
	kfacInfo->dampGamma = 100;
	kfacInfo->checkGrad = 1;
	kfacInfo->inverseFreq = 1;
}

int kfacParamsFileName(CNN_MODEL *model, int dataset, int initialization, char *out, int outBytes)
{
	static const char *folders[3] = { "cifar10/", "cifar100/", "imagenet/" };
	static const char *inits[3] = { "default", "kaiming", "xavier" };
	const char *net;
	switch (model->name) {
	case CNN_LENET: net = "lenet"; break;
	case CNN_ALEXNET: net = "alexnet"; break;
	case CNN_VGG11NET: net = "vgg11"; break;
	case CNN_VGG13NET: net = "vgg13"; break;
	case CNN_VGG16NET: net = "vgg16"; break;
	case CNN_VGG19NET: net = "vgg19"; break;
	default: return -1;
	}
	if (dataset < 1 || dataset > 3 || initialization < 0 || initialization > 2) return -1;
	int n = snprintf(out, (size_t)outBytes, "%s%s%s_%s%s.params", weights_folder(), folders[dataset - 1], net,
	                 inits[initialization], model->bias != 0 ? "_bias" : "");
	return n > 0 && n < outBytes ? 0 : -1;
}

void testKFACTrustRegion(CNN_MODEL *model, DEVICE_DATASET *data, HOST_DATASET *host, SCRATCH_AREA *scratch, real dampGamma,
                         real trMaxRadius, int checkGrad, int master, int slave, int inverseFreq, int epochs, int dataset,
                         real regLambda, int initialization)
{
	char paramsFile[PATH_BYTES];
	TRUST_REGION_PARAMS trParams;
	KFAC_CURVATURE_INFO kfacInfo;

	fprintf(stderr, "Initiating the Trust Region Test now..... \n\n\n");
	initKFACTrustRegionParams(&trParams, data->trainSizeX);
	initKFACInfo(&kfacInfo);
	kfacInfo.dampGamma = dampGamma;
	kfacInfo.checkGrad = checkGrad;
	kfacInfo.inverseFreq = inverseFreq;
	kfacInfo.regLambda = regLambda;
	trParams.maxDelta = trMaxRadius;
	trParams.maxIters = epochs;
	data->sampleSize = data->trainSizeX;

	if (kfacParamsFileName(model, dataset, initialization, paramsFile, PATH_BYTES) != 0) {
		fprintf(stderr, "Unknown dataset (%d), network (%d) or initialization (%d) for the parameter file... \n", dataset,
		        (int)model->name, initialization);
		exit(-1);
	}
	fprintf(stderr, "Reading the params file: %s \n", paramsFile);
	int got = readVector(scratch->nextHostPtr, model->pSize, paramsFile, 0, NULL);
	if (got != model->pSize) {
		fprintf(stderr, "testKFACTrustRegion: %s holds %d values, the network has %d parameters\n", paramsFile, got,
		        model->pSize);
		exit(-1);
	}
	copy_host_device(scratch->nextHostPtr, data->weights, sizeof(real) * (size_t)model->pSize, cudaMemcpyHostToDevice,
	                 ERROR_MEMCPY_HOST_DEVICE);

	fprintf(stderr, "Starting the KFAC Algorithm now.... \n");
	subsampledTrustRegionKFAC(model, data, host, &kfacInfo, &trParams, scratch, master, slave);
	fprintf(stderr, ".... Done testing of KFAC Trust Region Done. \n\n\n");
}
