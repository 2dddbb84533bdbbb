/*
 * A driver in the shape of the reference's own (drivers/main_driver.c:62-305, test 8): it is written against
 * the reference's function names and links the two libraries instead of the reference's sources.  The one
 * departure: the device arena is sized with kfacTrustRegionMemRequired instead of taking all free memory
 * (cuda_allocate_workspace, which is there too).
 *
 *   kfac_driver <dataset 1|2|3> <network 1|2|3> <epochs> <dampGamma> <maxRadius> <inverseFreq> <regLambda>
 *               <initialization 0|1|2> <dataset folder> <weights folder>
 *
 * Without arguments it prints this usage and exits with status 2 before anything touches a device.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "fitre_cnn.h"
#include "fitre_dataset.h"
#include "fitre_shim.h"

int main(int argc, char **argv)
{
	if (argc != 11) {
		fprintf(stderr, "usage: %s dataset network epochs dampGamma maxRadius inverseFreq regLambda initialization "
		                "datasetFolder weightsFolder\n", argv[0]);
		return 2;
	}
	const int dataset = atoi(argv[1]), network = atoi(argv[2]), epochs = atoi(argv[3]);
	const real dampGamma = (real)atof(argv[4]), maxRadius = (real)atof(argv[5]);
	const int inverseFreq = atoi(argv[6]);
	const real regLambda = (real)atof(argv[7]);
	const int initialization = atoi(argv[8]);
	const int batch = 256;

	SCRATCH_AREA scratch;
	HOST_DATASET hostData;
	DEVICE_DATASET deviceData;
	CNN_MODEL model;
	memset(&hostData, 0, sizeof hostData);
	memset(&deviceData, 0, sizeof deviceData);
	memset(&model, 0, sizeof model);

	getDeviceParameters();
	cuda_env_init(&scratch, 0);
	fitreSetDatasetFolder(dataset, argv[9]);
	fitreSetWeightsFolder(argv[10]);
	model.batchSize = batch;
	switch (dataset) {
	case 1: getCIFAR10(&model, &hostData, &deviceData, &scratch); break;
	case 2: getCIFAR100(&model, &hostData, &deviceData, &scratch); break;
	case 3: getTinyImageNet(&model, &hostData, &deviceData, &scratch); break;
	default: fprintf(stderr, " Unknown dataset parameter: %d \n", dataset); return 1;
	}
	switch (network) {
	case 1: readLenetCNN(&model, 3, deviceData.width, deviceData.height, batch, 1, 1); break;
	case 2: readAlexNetCNN(&model, batch, deviceData.height, deviceData.width, deviceData.numClasses, 1, 1); break;
	case 3: readVGG11(&model, batch, deviceData.height, deviceData.width, deviceData.numClasses, 3, 1, 1, hostData.datasetType); break;
	default: fprintf(stderr, "Unknown NETWORK Name: %d \n", network); return 1;
	}
	cnnInitializations(&model, &deviceData);
	KFAC_CURVATURE_INFO sizing;
	initKFACInfo(&sizing);
	sizing.inverseFreq = inverseFreq;
	fitre_allocate_workspace(&scratch, sizeof(real) * (size_t)kfacTrustRegionMemRequired(&model, &deviceData, &sizing));
	testKFACTrustRegion(&model, &deviceData, &hostData, &scratch, dampGamma, maxRadius, 0, 0, 0, inverseFreq, epochs, dataset,
	                    regLambda, initialization);
	cleanup_dataset(&hostData, &deviceData);
	cuda_env_cleanup(&scratch);
	return 0;
}
