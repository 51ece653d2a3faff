// Hand-written declarations for the subset of the isl C API (integer set library,
// MIT licence) that the front-end and the AST layer call.  The image ships the
// runtime library libisl.so.23 (isl 0.24) without headers, so the prototypes are
// declared here and the library is linked by file name.  All isl objects are
// opaque pointers; enum values below are part of isl's stable ABI.
#ifndef TIRAMISU_AMD_ISL_API_H
#define TIRAMISU_AMD_ISL_API_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct isl_ctx isl_ctx;
typedef struct isl_set isl_set;
typedef struct isl_basic_set isl_basic_set;
typedef struct isl_map isl_map;
typedef struct isl_basic_map isl_basic_map;
typedef struct isl_union_set isl_union_set;
typedef struct isl_union_map isl_union_map;
typedef struct isl_space isl_space;
typedef struct isl_local_space isl_local_space;
typedef struct isl_id isl_id;
typedef struct isl_id_list isl_id_list;
typedef struct isl_val isl_val;
typedef struct isl_aff isl_aff;
typedef struct isl_pw_aff isl_pw_aff;
typedef struct isl_multi_aff isl_multi_aff;
typedef struct isl_pw_multi_aff isl_pw_multi_aff;
typedef struct isl_ast_build isl_ast_build;
typedef struct isl_ast_node isl_ast_node;
typedef struct isl_ast_node_list isl_ast_node_list;
typedef struct isl_ast_expr isl_ast_expr;
typedef struct isl_constraint isl_constraint;
typedef struct isl_map_list isl_map_list;
typedef struct isl_schedule isl_schedule;
typedef struct isl_schedule_node isl_schedule_node;
typedef struct isl_union_set_list isl_union_set_list;
typedef struct isl_union_pw_aff isl_union_pw_aff;
typedef struct isl_multi_union_pw_aff isl_multi_union_pw_aff;

typedef int isl_size;
typedef enum { isl_bool_error = -1, isl_bool_false = 0, isl_bool_true = 1 } isl_bool;
typedef enum { isl_stat_error = -1, isl_stat_ok = 0 } isl_stat;

enum isl_dim_type { isl_dim_cst, isl_dim_param, isl_dim_in, isl_dim_out,
                    isl_dim_set = isl_dim_out, isl_dim_div, isl_dim_all };

enum isl_ast_node_type { isl_ast_node_error = -1, isl_ast_node_for = 1, isl_ast_node_if,
                         isl_ast_node_block, isl_ast_node_mark, isl_ast_node_user };

enum isl_ast_expr_type { isl_ast_expr_error = -1, isl_ast_expr_op, isl_ast_expr_id,
                         isl_ast_expr_int };

enum isl_ast_op_type {
    isl_ast_op_error = -1, isl_ast_op_and, isl_ast_op_and_then, isl_ast_op_or,
    isl_ast_op_or_else, isl_ast_op_max, isl_ast_op_min, isl_ast_op_minus, isl_ast_op_add,
    isl_ast_op_sub, isl_ast_op_mul, isl_ast_op_div, isl_ast_op_fdiv_q, isl_ast_op_pdiv_q,
    isl_ast_op_pdiv_r, isl_ast_op_zdiv_r, isl_ast_op_cond, isl_ast_op_select, isl_ast_op_eq,
    isl_ast_op_le, isl_ast_op_lt, isl_ast_op_ge, isl_ast_op_gt, isl_ast_op_call,
    isl_ast_op_access, isl_ast_op_member, isl_ast_op_address_of
};

#define ISL_ON_ERROR_WARN 0
#define ISL_ON_ERROR_CONTINUE 1
#define ISL_ON_ERROR_ABORT 2

// context and options
isl_ctx *isl_ctx_alloc(void);
void isl_ctx_free(isl_ctx *ctx);
isl_stat isl_options_set_on_error(isl_ctx *ctx, int val);
isl_stat isl_options_set_ast_build_atomic_upper_bound(isl_ctx *ctx, int val);
isl_stat isl_options_set_ast_build_group_coscheduled(isl_ctx *ctx, int val);
isl_stat isl_options_set_ast_build_exploit_nested_bounds(isl_ctx *ctx, int val);
isl_stat isl_options_set_ast_build_allow_else(isl_ctx *ctx, int val);
void isl_ctx_reset_error(isl_ctx *ctx);

// identifiers and values
isl_id *isl_id_alloc(isl_ctx *ctx, const char *name, void *user);
const char *isl_id_get_name(isl_id *id);
void *isl_id_get_user(isl_id *id);
isl_id *isl_id_free(isl_id *id);
isl_id_list *isl_id_list_alloc(isl_ctx *ctx, int n);
isl_id_list *isl_id_list_add(isl_id_list *list, isl_id *el);
long isl_val_get_num_si(isl_val *v);
long isl_val_get_den_si(isl_val *v);
isl_bool isl_val_is_int(isl_val *v);
isl_val *isl_val_free(isl_val *v);

// spaces
isl_space *isl_space_free(isl_space *space);
isl_space *isl_space_params_alloc(isl_ctx *ctx, unsigned nparam);

// sets
isl_set *isl_set_read_from_str(isl_ctx *ctx, const char *str);
isl_set *isl_set_copy(isl_set *set);
isl_set *isl_set_free(isl_set *set);
char *isl_set_to_str(isl_set *set);
isl_size isl_set_dim(isl_set *set, enum isl_dim_type type);
const char *isl_set_get_dim_name(isl_set *set, enum isl_dim_type type, unsigned pos);
const char *isl_set_get_tuple_name(isl_set *set);
isl_set *isl_set_set_tuple_name(isl_set *set, const char *s);
isl_set *isl_set_set_dim_name(isl_set *set, enum isl_dim_type type, unsigned pos, const char *s);
isl_set *isl_set_intersect(isl_set *a, isl_set *b);
isl_set *isl_set_intersect_params(isl_set *set, isl_set *params);
isl_set *isl_set_subtract(isl_set *a, isl_set *b);
isl_set *isl_set_union(isl_set *a, isl_set *b);
isl_set *isl_set_coalesce(isl_set *set);
isl_set *isl_set_apply(isl_set *set, isl_map *map);
isl_bool isl_set_is_empty(isl_set *set);
isl_bool isl_set_is_equal(isl_set *a, isl_set *b);
isl_bool isl_set_is_subset(isl_set *a, isl_set *b);
isl_space *isl_set_get_space(isl_set *set);
isl_set *isl_set_project_out(isl_set *set, enum isl_dim_type type, unsigned first, unsigned n);
isl_set *isl_set_params(isl_set *set);
isl_ctx *isl_set_get_ctx(isl_set *set);
isl_val *isl_set_dim_max_val(isl_set *set, int pos);
isl_val *isl_set_dim_min_val(isl_set *set, int pos);
isl_set *isl_set_align_params(isl_set *set, isl_space *model);
isl_set *isl_set_lexmin(isl_set *set);
isl_set *isl_set_lexmax(isl_set *set);
isl_bool isl_set_is_singleton(isl_set *set);
isl_val *isl_set_plain_get_val_if_fixed(isl_set *set, enum isl_dim_type type, unsigned pos);
isl_val *isl_set_count_val(isl_set *set);
isl_bool isl_set_plain_is_universe(isl_set *set);
isl_size isl_pw_aff_n_piece(isl_pw_aff *pwaff);
isl_set *isl_set_remove_redundancies(isl_set *set);

// maps
isl_map *isl_map_read_from_str(isl_ctx *ctx, const char *str);
isl_map *isl_map_copy(isl_map *map);
isl_map *isl_map_free(isl_map *map);
char *isl_map_to_str(isl_map *map);
isl_size isl_map_dim(isl_map *map, enum isl_dim_type type);
const char *isl_map_get_tuple_name(isl_map *map, enum isl_dim_type type);
isl_map *isl_map_set_tuple_name(isl_map *map, enum isl_dim_type type, const char *s);
const char *isl_map_get_dim_name(isl_map *map, enum isl_dim_type type, unsigned pos);
isl_map *isl_map_apply_range(isl_map *a, isl_map *b);
isl_map *isl_map_apply_domain(isl_map *a, isl_map *b);
isl_map *isl_map_intersect(isl_map *a, isl_map *b);
isl_map *isl_map_intersect_domain(isl_map *map, isl_set *set);
isl_map *isl_map_intersect_range(isl_map *map, isl_set *set);
isl_map *isl_map_intersect_params(isl_map *map, isl_set *params);
isl_map *isl_map_reverse(isl_map *map);
isl_set *isl_map_domain(isl_map *map);
isl_set *isl_map_range(isl_map *map);
isl_map *isl_map_project_out(isl_map *map, enum isl_dim_type type, unsigned first, unsigned n);
isl_map *isl_map_add_dims(isl_map *map, enum isl_dim_type type, unsigned n);
isl_map *isl_map_fix_si(isl_map *map, enum isl_dim_type type, unsigned pos, int value);
isl_bool isl_map_is_single_valued(isl_map *map);
isl_bool isl_map_is_empty(isl_map *map);
isl_bool isl_map_is_equal(isl_map *a, isl_map *b);
isl_bool isl_map_is_subset(isl_map *a, isl_map *b);
isl_map *isl_map_range_product(isl_map *a, isl_map *b);
isl_map *isl_map_equate(isl_map *map, enum isl_dim_type type1, int pos1, enum isl_dim_type type2, int pos2);
isl_val *isl_map_plain_get_val_if_fixed(isl_map *map, enum isl_dim_type type, unsigned pos);
isl_space *isl_map_get_space(isl_map *map);
isl_map *isl_map_coalesce(isl_map *map);
isl_map *isl_map_align_params(isl_map *map, isl_space *model);
isl_map *isl_map_union(isl_map *a, isl_map *b);
isl_map *isl_map_lexmin(isl_map *map);
isl_map *isl_map_lexmax(isl_map *map);
isl_set *isl_map_deltas(isl_map *map);
isl_bool isl_map_involves_dims(isl_map *map, enum isl_dim_type type, unsigned first, unsigned n);
isl_map *isl_set_identity(isl_set *set);

// union sets and maps
isl_union_map *isl_union_map_from_map(isl_map *map);
isl_union_map *isl_union_map_union(isl_union_map *a, isl_union_map *b);
isl_union_map *isl_union_map_copy(isl_union_map *umap);
isl_union_map *isl_union_map_free(isl_union_map *umap);
isl_union_map *isl_union_map_read_from_str(isl_ctx *ctx, const char *str);
char *isl_union_map_to_str(isl_union_map *umap);
isl_map *isl_map_from_union_map(isl_union_map *umap);
isl_union_map *isl_union_map_intersect_domain(isl_union_map *umap, isl_union_set *uset);
isl_union_set *isl_union_set_from_set(isl_set *set);
isl_union_set *isl_union_set_union(isl_union_set *a, isl_union_set *b);
isl_union_set *isl_union_map_domain(isl_union_map *umap);
isl_map_list *isl_union_map_get_map_list(isl_union_map *umap);
isl_size isl_map_list_n_map(isl_map_list *list);
isl_map *isl_map_list_get_map(isl_map_list *list, int index);
isl_map_list *isl_map_list_free(isl_map_list *list);
isl_bool isl_union_map_is_equal(isl_union_map *a, isl_union_map *b);

/* dataflow analysis: the last write (must source) that every read (sink) sees under a schedule */
typedef struct isl_union_access_info isl_union_access_info;
typedef struct isl_union_flow isl_union_flow;
isl_union_access_info *isl_union_access_info_from_sink(isl_union_map *sink);
isl_union_access_info *isl_union_access_info_set_must_source(isl_union_access_info *access, isl_union_map *must_source);
isl_union_access_info *isl_union_access_info_set_schedule_map(isl_union_access_info *access, isl_union_map *schedule_map);
isl_union_flow *isl_union_access_info_compute_flow(isl_union_access_info *access);
isl_union_map *isl_union_flow_get_must_dependence(isl_union_flow *flow);
isl_union_access_info *isl_union_access_info_set_may_source(isl_union_access_info *access, isl_union_map *may_source);
isl_union_access_info *isl_union_access_info_set_kill(isl_union_access_info *access, isl_union_map *kill);
/* { source -> [sink -> memory cell] }: the dependence together with the cell it goes through */
isl_union_map *isl_union_flow_get_full_must_dependence(isl_union_flow *flow);
isl_union_map *isl_union_flow_get_full_may_dependence(isl_union_flow *flow);
/* the sink accesses that no source writes before them */
isl_union_map *isl_union_flow_get_must_no_source(isl_union_flow *flow);
isl_union_map *isl_union_map_range_factor_domain(isl_union_map *umap);
isl_union_map *isl_union_map_range_factor_range(isl_union_map *umap);
isl_union_map *isl_union_map_subtract(isl_union_map *a, isl_union_map *b);
isl_union_map *isl_union_map_apply_range(isl_union_map *a, isl_union_map *b);
isl_union_map *isl_union_map_apply_domain(isl_union_map *a, isl_union_map *b);
isl_union_map *isl_union_map_intersect_range(isl_union_map *umap, isl_union_set *uset);
isl_union_map *isl_union_map_coalesce(isl_union_map *umap);
isl_bool isl_union_map_is_empty(isl_union_map *umap);
isl_stat isl_union_map_foreach_map(isl_union_map *umap, isl_stat (*fn)(isl_map *map, void *user), void *user);
isl_stat isl_map_foreach_basic_map(isl_map *map, isl_stat (*fn)(isl_basic_map *bmap, void *user), void *user);
isl_map *isl_map_from_basic_map(isl_basic_map *bmap);
isl_map *isl_map_lex_ge(isl_space *set_space);
isl_space *isl_space_range(isl_space *space);
isl_set *isl_map_params(isl_map *map);
isl_map *isl_map_subtract(isl_map *a, isl_map *b);
isl_union_flow *isl_union_flow_free(isl_union_flow *flow);
isl_union_set *isl_union_set_free(isl_union_set *uset);
isl_union_set *isl_union_set_copy(isl_union_set *uset);
isl_union_map *isl_union_map_reverse(isl_union_map *umap);

// piecewise affine functions
isl_pw_multi_aff *isl_pw_multi_aff_from_map(isl_map *map);
isl_pw_multi_aff *isl_pw_multi_aff_free(isl_pw_multi_aff *pma);
isl_pw_aff *isl_pw_multi_aff_get_pw_aff(isl_pw_multi_aff *pma, int pos);
isl_size isl_pw_multi_aff_dim(isl_pw_multi_aff *pma, enum isl_dim_type type);
isl_pw_aff *isl_pw_aff_free(isl_pw_aff *pa);
isl_pw_aff *isl_set_dim_max(isl_set *set, int pos);
isl_pw_aff *isl_set_dim_min(isl_set *set, int pos);
char *isl_pw_aff_to_str(isl_pw_aff *pa);

// AST generation
isl_ast_build *isl_ast_build_alloc(isl_ctx *ctx);
isl_ast_build *isl_ast_build_from_context(isl_set *set);
isl_ast_build *isl_ast_build_free(isl_ast_build *build);
isl_ast_build *isl_ast_build_set_at_each_domain(isl_ast_build *build,
        isl_ast_node *(*fn)(isl_ast_node *node, isl_ast_build *build, void *user), void *user);
isl_ast_build *isl_ast_build_set_iterators(isl_ast_build *build, isl_id_list *iterators);
isl_ast_node *isl_ast_build_node_from_schedule_map(isl_ast_build *build, isl_union_map *schedule);
isl_union_map *isl_ast_build_get_schedule(isl_ast_build *build);
isl_ast_expr *isl_ast_build_access_from_pw_multi_aff(isl_ast_build *build, isl_pw_multi_aff *pma);
isl_ast_expr *isl_ast_build_call_from_pw_multi_aff(isl_ast_build *build, isl_pw_multi_aff *pma);
isl_ast_expr *isl_ast_build_expr_from_pw_aff(isl_ast_build *build, isl_pw_aff *pa);

// schedule trees (the second way into the AST generator)
isl_schedule *isl_schedule_from_domain(isl_union_set *domain);
isl_schedule *isl_schedule_free(isl_schedule *schedule);
isl_schedule *isl_schedule_copy(isl_schedule *schedule);
isl_schedule_node *isl_schedule_get_root(isl_schedule *schedule);
isl_schedule *isl_schedule_node_get_schedule(isl_schedule_node *node);
isl_schedule_node *isl_schedule_node_free(isl_schedule_node *node);
isl_schedule_node *isl_schedule_node_child(isl_schedule_node *node, int pos);
isl_schedule_node *isl_schedule_node_parent(isl_schedule_node *node);
isl_schedule_node *isl_schedule_node_insert_sequence(isl_schedule_node *node, isl_union_set_list *filters);
isl_schedule_node *isl_schedule_node_insert_partial_schedule(isl_schedule_node *node, isl_multi_union_pw_aff *schedule);
isl_union_set_list *isl_union_set_list_alloc(isl_ctx *ctx, int n);
isl_union_set_list *isl_union_set_list_add(isl_union_set_list *list, isl_union_set *el);
isl_union_pw_aff *isl_union_pw_aff_from_pw_aff(isl_pw_aff *pa);
isl_union_pw_aff *isl_union_pw_aff_union_add(isl_union_pw_aff *a, isl_union_pw_aff *b);
isl_multi_union_pw_aff *isl_multi_union_pw_aff_from_union_pw_aff(isl_union_pw_aff *upa);
isl_ast_node *isl_ast_build_node_from_schedule(isl_ast_build *build, isl_schedule *schedule);

enum isl_ast_node_type isl_ast_node_get_type(isl_ast_node *node);
isl_ast_expr *isl_ast_node_for_get_iterator(isl_ast_node *node);
isl_ast_expr *isl_ast_node_for_get_init(isl_ast_node *node);
isl_ast_expr *isl_ast_node_for_get_cond(isl_ast_node *node);
isl_ast_expr *isl_ast_node_for_get_inc(isl_ast_node *node);
isl_ast_node *isl_ast_node_for_get_body(isl_ast_node *node);
isl_bool isl_ast_node_for_is_degenerate(isl_ast_node *node);
isl_ast_expr *isl_ast_node_if_get_cond(isl_ast_node *node);
isl_ast_node *isl_ast_node_if_get_then(isl_ast_node *node);
isl_ast_node *isl_ast_node_if_get_else(isl_ast_node *node);
isl_bool isl_ast_node_if_has_else(isl_ast_node *node);
isl_ast_node_list *isl_ast_node_block_get_children(isl_ast_node *node);
isl_ast_node *isl_ast_node_mark_get_node(isl_ast_node *node);
isl_ast_expr *isl_ast_node_user_get_expr(isl_ast_node *node);
isl_ast_node *isl_ast_node_set_annotation(isl_ast_node *node, isl_id *annotation);
isl_id *isl_ast_node_get_annotation(isl_ast_node *node);
isl_ast_node *isl_ast_node_free(isl_ast_node *node);
char *isl_ast_node_to_C_str(isl_ast_node *node);
isl_size isl_ast_node_list_n_ast_node(isl_ast_node_list *list);
isl_ast_node *isl_ast_node_list_get_ast_node(isl_ast_node_list *list, int index);
isl_ast_node_list *isl_ast_node_list_free(isl_ast_node_list *list);

enum isl_ast_expr_type isl_ast_expr_get_type(isl_ast_expr *expr);
enum isl_ast_op_type isl_ast_expr_get_op_type(isl_ast_expr *expr);
isl_size isl_ast_expr_get_op_n_arg(isl_ast_expr *expr);
isl_ast_expr *isl_ast_expr_get_op_arg(isl_ast_expr *expr, int pos);
isl_id *isl_ast_expr_get_id(isl_ast_expr *expr);
isl_val *isl_ast_expr_get_val(isl_ast_expr *expr);
isl_ast_expr *isl_ast_expr_free(isl_ast_expr *expr);
char *isl_ast_expr_to_C_str(isl_ast_expr *expr);

#ifdef __cplusplus
}
#endif
#endif
