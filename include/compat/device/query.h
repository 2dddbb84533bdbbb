/* device/query.h of the reference: getDeviceParameters (device/query.h) */
#include "fitre_shim.h"
