/*
 * Compile-only check (test infrastructure): the reference's libnc.h is
 * included first, then this repository's headers.  Any prototype of
 * nc_api.h that disagreed with the reference declaration of the same name
 * would be a "conflicting types" error, and the static assertions pin the
 * layout of the public structs the host code reads directly.
 */
#include <stdio.h>
#include "libnc.h"            /* the reference header, found through -I */
#include "../include/nc_api.h"
#include "../include/nc_ext.h"

_Static_assert(sizeof(SGDOptParams) == 32, "SGDOptParams layout");
_Static_assert(sizeof(NCParamList) == sizeof(void *) * 4, "NCParamList layout");
_Static_assert(NC_TYPE_I32 == 5 && NC_TYPE_U16 == 7, "NCTypeEnum values");

int nc_abi_check_dummy;
