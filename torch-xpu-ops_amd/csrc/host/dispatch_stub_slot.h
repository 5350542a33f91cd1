// Reading and replacing the GPU slot of one of ATen's DispatchStub objects.
//
// ATen gives a DispatchStub a setter for its GPU kernel (set_cuda_dispatch_ptr;
// the "cuda" slot is the HIP one in a ROCm build) but no getter, and putting the
// stock kernel back on uninstall -- or handing float64 calls on to it -- needs the
// previous value.  It is read through the object's layout: a DispatchStub<fn, T>
// is a standard-layout class whose only non-static data member is its
// DispatchStubImpl (ATen/native/DispatchStub.h; checked against PyTorch 2.10.0,
// the version this library is built and tested with), so the object's address is
// that member's address.  That layout is private to ATen and may change between
// PyTorch builds, so it is guarded three ways: the compile-time checks below, a
// run-time check that the slot read this way really is the one the setter writes
// (install_checked() installs, reads back, and refuses -- restoring what it found
// -- if the two disagree), and the uninstall going through the same setter.
#pragma once
#include <ATen/native/DispatchStub.h>
#include <c10/util/Exception.h>

#include <type_traits>

namespace mi355x {

template <class Stub>
void* gpu_slot_value(Stub& stub) {
  static_assert(std::is_standard_layout<Stub>::value,
                "DispatchStub is no longer a standard-layout class: its first member's address "
                "is not the object's");
  static_assert(sizeof(Stub) == sizeof(at::native::DispatchStubImpl),
                "DispatchStub holds more than its DispatchStubImpl");
  return reinterpret_cast<at::native::DispatchStubImpl*>(&stub)->cuda_dispatch_ptr;
}

// Installs `fn` as the GPU kernel of `stub`; returns the kernel that was there.
template <class Stub, class Fn>
void* install_checked(Stub& stub, Fn* fn, const char* name) {
  void* previous = gpu_slot_value(stub);
  stub.set_cuda_dispatch_ptr(fn);
  if (gpu_slot_value(stub) != reinterpret_cast<void*>(fn)) {
    // the layout assumption does not hold in this PyTorch build: `previous` is not the
    // slot's old value either, so nothing can be restored but nothing is kept installed
    // under a wrong belief; the process keeps running with the stub as the setter left it
    TORCH_CHECK(false, "mi355x: cannot read the GPU slot of ATen's ", name,
                " dispatch stub in this PyTorch build (DispatchStub layout differs from the "
                "2.10 one this library was checked against); the stub now points at the MI355X "
                "kernel and cannot be uninstalled");
  }
  return previous;
}

template <class Stub, class Fn>
void restore(Stub& stub, void* previous) {
  stub.set_cuda_dispatch_ptr(reinterpret_cast<Fn*>(previous));
}

}  // namespace mi355x
