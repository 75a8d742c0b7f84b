#include "frontend/reduce_split_pass.h"

#include <algorithm>
#include <map>

#include "frontend/pass_util.h"

namespace cinn {
namespace frontend {

namespace {

using hlir::framework::GetAttr;
using utils::AttributeMap;
using utils::ShapeType;

const std::map<std::string, std::string>& ReduceKinds() {
  static const std::map<std::string, std::string> kinds = {{"reduce_sum", "sum"}, {"reduce_prod", "prod"},
                                                           {"reduce_max", "max"}, {"reduce_min", "min"},
                                                           {"reduce_all", "all"}, {"reduce_any", "any"}};
  return kinds;
}

int64_t Product(const std::vector<int64_t>& v, size_t begin, size_t end) {
  int64_t p = 1;
  for (size_t i = begin; i < end; ++i) p *= v[i];
  return p;
}

// slices of r for a column reduce of [a][r][c]: the smallest divisor of r that gives the kernel about four blocks
// per compute unit while every block still walks at least min_rows rows; 1 when the grid is large enough already
int ChooseParts(int64_t a, int64_t r, int64_t c, int elem_bytes, int num_compute_units, int64_t min_rows = 32) {
  int vec = std::max(1, std::min(16 / elem_bytes, 8));
  while (vec > 1 && c % vec != 0) vec /= 2;
  const int64_t column_blocks = (c / vec + 63) / 64;
  const int64_t blocks        = a * column_blocks;
  const int64_t wanted        = static_cast<int64_t>(num_compute_units) * 4;
  if (blocks >= wanted || r < 2 * min_rows) return 1;
  int best = 1;
  for (int64_t d = 2; d <= r / min_rows && d <= 4096; ++d) {
    if (r % d != 0) continue;
    best = static_cast<int>(d);
    if (blocks * d >= wanted) break;
  }
  return best;
}

}  // namespace

Program SplitReductions(const Program& program, int num_compute_units) {
  std::vector<Instruction> out;
  Emitter emit(&out, "rsplit_");
  for (auto& ins : program.instructions()) {
    auto kind_it = ReduceKinds().find(ins->op_type);
    if (kind_it == ReduceKinds().end()) {
      out.push_back(ins);
      continue;
    }
    const std::string& kind = kind_it->second;
    const Variable& x       = ins->inputs[0];
    const Variable& y       = ins->outputs[0];
    const int rank          = static_cast<int>(x->shape.size());
    auto dims               = GetAttr<std::vector<int>>(ins->attrs, "dim", {});
    std::vector<bool> reduced(rank, dims.empty());
    for (int d : dims) reduced[d < 0 ? d + rank : d] = true;

    // the shape without its axes of size 1, which belong to no run
    std::vector<int64_t> sq;
    std::vector<bool> sq_reduced;
    std::vector<int> sq_axis;  // axis of x
    for (int i = 0; i < rank; ++i) {
      if (x->shape[i] == 1) continue;
      sq.push_back(x->shape[i]);
      sq_reduced.push_back(reduced[i]);
      sq_axis.push_back(i);
    }
    std::vector<std::pair<size_t, size_t>> runs;  // [begin, end) in sq
    for (size_t i = 0; i < sq.size();) {
      if (!sq_reduced[i]) {
        ++i;
        continue;
      }
      size_t j = i;
      while (j < sq.size() && sq_reduced[j]) ++j;
      runs.push_back({i, j});
      i = j;
    }
    const bool trailing_only = runs.size() == 1 && runs[0].second == sq.size();
    // a few very long rows (a full reduction is one row): the row-reduce template would give each row to a single
    // block, so slices of the row are reduced first, as a [a][parts][r / parts][1] run
    int row_parts = 1;
    if (trailing_only) {
      const int64_t a = Product(sq, 0, runs[0].first), r = Product(sq, runs[0].first, sq.size());
      // measured: one block per row takes about 10 us per 64 Ki elements of a row; the sliced form costs two extra
      // launches and, in a fused group, a second pass over the input
      const bool few_rows = a < num_compute_units && (r >= 131072 || (a <= 16 && r >= 65536));
      if (few_rows) row_parts = ChooseParts(a, r, 1, x->type.bytes(), num_compute_units, 4096);
    }
    if (runs.empty() || (trailing_only && row_parts == 1)) {
      out.push_back(ins);
      continue;
    }

    const bool wide_partials = (kind == "sum" || kind == "prod") && (x->type.is_float16() || x->type.is_bfloat16());
    const std::string partial_type = wide_partials ? "float32" : "";
    const std::string final_type   = common::Type2Str(y->type);
    Variable cur                   = x;
    bool cur_is_x                  = true;
    auto to_shape                  = [](const std::vector<int64_t>& v) {
      ShapeType s;
      for (int64_t d : v) s.push_back(static_cast<int>(d));
      if (s.empty()) s.push_back(1);
      return s;
    };
    // one reduce_run step over sq[begin, end), leaving `parts` slices; the last step defines y itself
    auto run_step = [&](size_t begin, size_t end, int parts, bool last) {
      const int64_t a = Product(sq, 0, begin), r = Product(sq, begin, end), c = Product(sq, end, sq.size());
      std::vector<int64_t> next(sq.begin(), sq.begin() + begin);
      if (parts > 1) next.push_back(parts);
      next.insert(next.end(), sq.begin() + end, sq.end());
      AttributeMap attrs = {{"a", static_cast<int>(a)},
                            {"r", static_cast<int>(r)},
                            {"c", static_cast<int>(c)},
                            {"parts", parts},
                            {"out_shape", last ? y->shape : to_shape(next)},
                            {"dtype", last ? final_type : partial_type}};
      const std::string op = "reduce_run_" + kind;
      if (last) {
        emit.EmitInto(y, op, {cur}, attrs);
      } else {
        cur      = emit.Emit1(op, {cur}, attrs);
        cur_is_x = false;
      }
      sq = next;
    };
    for (size_t ri = runs.size(); ri-- > 0;) {
      const size_t begin = runs[ri].first, end = runs[ri].second;
      const bool first_run = ri == 0;  // processed last
      if (end == sq.size() && cur_is_x && !trailing_only) {
        // the trailing run: an ordinary reduction over the last axes (row-reduce template)
        std::vector<int> axes;
        for (size_t i = begin; i < end; ++i) axes.push_back(sq_axis[i]);
        cur      = emit.Emit1(ins->op_type, {cur}, {{"dim", axes}, {"keep_dim", false}});
        cur_is_x = false;
        sq.erase(sq.begin() + begin, sq.begin() + end);
        continue;
      }
      const int64_t a = Product(sq, 0, begin), r = Product(sq, begin, end), c = Product(sq, end, sq.size());
      const int parts = trailing_only ? row_parts : ChooseParts(a, r, c, x->type.bytes(), num_compute_units);
      run_step(begin, end, parts, first_run && parts == 1);
      if (parts > 1) run_step(begin, begin + 1, 1, first_run);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

}  // namespace frontend
}  // namespace cinn
