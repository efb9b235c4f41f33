"""TEST INFRASTRUCTURE ONLY: the CPU oracle for the GPT-2 training kernels.

c_oracle   - ctypes front end of oracle/_build/libcs_oracle.so (cs_oracle.c,
             the scalar C restatement of the reference's task bodies)
aten_port  - the reference's own op sequences, issued to the installed ATen
             CPU kernels (the library its task bodies call)

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this package.  Nothing under core_scheduler_amd/ does.
"""
