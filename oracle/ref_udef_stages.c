/*
 * ref_udef_stages.c -- the caller's side of a reference build in which all five
 * stages may be user functions.  Test infrastructure only.
 *
 * Built by oracle/Makefile together with /root/reference/fusedMM.c compiled
 * where it lies with -DVOP_UDEF_IMPL -DROP_UDEF_IMPL -DVSC_UDEF_IMPL
 * -DAOP_UDEF_IMPL (the switches of fusedMM.h:129-133; SOP_UDEF_IMPL is always
 * on there): the stubs of fusedMM_internal.h:50-84 then drop out of the
 * reference's object and its selectors (fusedMM.c:341-485) bind the functions
 * below.  This file contains no reference code.
 */
#include <stdint.h>

#ifndef INDEXTYPE
#error "build with -DINDEXTYPE=int32_t or int64_t"
#endif
#ifdef DREAL
#define VALUETYPE double
#else
#define VALUETYPE float
#endif

#define UDEF_IDX INDEXTYPE
#define UDEF_VAL VALUETYPE
#define UDEF_NAME(stage) stage##_UDEF_FUNC
#include "udef_stage_bodies.inc"

int ref_udef_index_bytes(void) { return (int)sizeof(INDEXTYPE); }
int ref_udef_value_bytes(void) { return (int)sizeof(VALUETYPE); }
