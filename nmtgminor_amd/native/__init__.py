"""Drop-in stand-ins for the reference's native extension modules (same names, same functions).

Each module validates its arguments the way the reference's C++ front end does (raising
RuntimeError), allocates the outputs the reference returns, and calls libnmtg_hip.so.
"""
