// EMPTY_TEMPLATE (empty_op.cc:3-53): the placeholder of a sub-matrix that contributes nothing to y.  It has no
// arrays and no kernel -- every code_of_* function of upstream's empty template returns an empty line -- so the
// builder launches nothing for it and clears y instead, which is what leaves its rows at zero.
// Upstream accepts a sub-block whose first and last element numbers are equal (empty_op.cc:13), which with its
// inclusive numbering is a block of one element that is then dropped from y; here the template takes a sub-matrix
// whose values are all zero (a strip of explicit zeros, the padding rows of a padded matrix), so that y = A x holds.
#include "templates.hpp"

namespace asx {
namespace tpl_empty {

bool is_supported(const Matrix &m, uint64_t sub) {
  const CompressedBlock &cb = *m.items[sub].cb;
  if (!cb.val) return true;
  for (double v : *cb.val)
    if (v != 0.0) return false;
  return true;
}

std::unique_ptr<Template> init(const Matrix &m, uint64_t sub) {
  AS_CHECK(is_supported(m, sub), "this sub dense block is not empty");
  auto t = std::make_unique<Template>();
  init_template_common(*t, EMPTY_TEMPLATE, m, sub);
  t->is_atom_add = false;
  t->col_index_arr.assign({}, UNSIGNED_CHAR);  // empty, but typed: the builder uploads every template's two arrays
  tpl_empty::set_default_launch(*t);
  return t;
}

void try_all_compress(Template &) {}

void set_default_launch(Template &t) {
  t.tblock_num = 1;  // nothing is launched; the launch-shape checks of the builder want a valid shape all the same
  t.thread_num_in_block = 64;
}

std::string kernel_source(const Template &t) {
  return "// sub-matrix " + std::to_string(t.sub) + ": no kernel\n";
}

}  // namespace tpl_empty
}  // namespace asx
