/* utilities/alloc_sampled_dataset.h of the reference: allocSampledDataset (utilities/alloc_sampled_dataset.h) */
#include "fitre_solver.h"
