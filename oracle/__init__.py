"""CPU oracle bindings (test infrastructure only).

`oracle.ep` wraps libtilexr_ep_oracle.so, the plain-C restatement of the reference's dispatch / combine
arithmetic; `oracle.ref` wraps _ref/libtilexr_ep_ref.so, the reference's own host sources compiled in
place (present only where the reference checkout was available at build time).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this package.
"""
