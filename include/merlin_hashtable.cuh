/*
 * The reference ships its public header under this name
 * (include/merlin_hashtable.cuh); callers that include it keep compiling.
 */
#include "merlin_hashtable.hpp"
