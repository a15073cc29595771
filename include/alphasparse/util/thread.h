/* Forwarding header: programs written against the reference's directory layout
 * (include/alphasparse/util/*.h) find the same declarations in alphasparse.h. */
#include "../../alphasparse.h"
