/* placeholder translation unit so the Makefile rule is stable; filled in with the cache model */
typedef int lxu_cache_model_placeholder_t;
