from . import build, build_stamped

build()
build_stamped()
