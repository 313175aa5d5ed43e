/* A few lines of "Lean runtime" for tests/test_lean_boundary.py only: enough to link the generated
 * weak stubs and read back the IO.userError message they build.  Objects are plain heap records. */
#include <lean/lean.h>
#include <stdlib.h>
#include <string.h>

struct lean_object { int kind; char* str; struct lean_object* inner; };   /* 1 string, 2 user error, 3 io error, 4 io ok */

static lean_object* mk(int kind, char* str, lean_object* inner) {
    lean_object* o = (lean_object*)malloc(sizeof(lean_object));
    o->kind = kind; o->str = str; o->inner = inner;
    return o;
}
lean_obj_res lean_mk_string(const char* s) { return mk(1, strdup(s), NULL); }
lean_obj_res lean_mk_io_user_error(lean_obj_arg str) { return mk(2, NULL, str); }
lean_obj_res lean_io_result_mk_error(lean_obj_arg e) { return mk(3, NULL, e); }
lean_obj_res lean_io_result_mk_ok(lean_obj_arg a) { return mk(4, NULL, a); }
lean_object* lean_box(size_t n) { (void)n; return mk(0, NULL, NULL); }

/* test accessors */
int tyr_test_is_io_error(lean_object* r) { return r && r->kind == 3 && r->inner && r->inner->kind == 2; }
const char* tyr_test_error_message(lean_object* r) { return tyr_test_is_io_error(r) ? r->inner->inner->str : NULL; }
