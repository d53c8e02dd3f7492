"""CPU oracle: test infrastructure only.  Never imported by diffcache_amd."""
