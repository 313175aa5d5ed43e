/* Declarations-only stand-in for <lean/lean.h>, used by tests/test_lean_boundary.py to type-check
 * tyr_amd/csrc/lean_shim.cpp and the emitted lean_launch_* wrappers where no Lean toolchain is
 * installed.  It declares exactly the runtime functions and object types those files use, with the
 * signatures Lean 4 documents for its C API (lean.h of the Lean 4 runtime): nothing here is ever
 * linked or executed, and nothing in the product includes it. */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lean_object lean_object;
typedef lean_object* lean_obj_arg;     /* owned argument    */
typedef lean_object* b_lean_obj_arg;   /* borrowed argument */
typedef lean_object* lean_obj_res;     /* owned result      */

lean_object* lean_alloc_ctor(unsigned tag, unsigned num_objs, unsigned scalar_sz);
void lean_ctor_set(lean_object* o, unsigned i, lean_obj_arg v);
lean_obj_res lean_io_result_mk_ok(lean_obj_arg a);
lean_obj_res lean_io_result_mk_error(lean_obj_arg e);
lean_obj_res lean_mk_io_user_error(lean_obj_arg str);
lean_obj_res lean_mk_string(const char* s);
lean_object* lean_box(size_t n);
lean_obj_res lean_box_uint64(uint64_t v);
lean_obj_res lean_box_float(double v);

#ifdef __cplusplus
}
#endif
